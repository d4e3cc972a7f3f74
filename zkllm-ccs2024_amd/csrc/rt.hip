// Runtime pieces of the C ABI: device selection, the caching allocator, copies, error text.
#include <cstdlib>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <utility>
#include <vector>
#include <cstdio>
#include <cstring>
#include "rt.hpp"
#include "field.hpp"
#include "../../include/zkllm_hip.h"

namespace zk {

static thread_local std::string g_err;
static thread_local int g_err_code = 0;

void set_error(int code, const std::string& msg) { g_err_code = code; g_err = msg; }
int hip_fail(hipError_t e, const char* what, const char* file, int line) {
    char buf[512];
    snprintf(buf, sizeof(buf), "%s failed: %s (%s:%d)", what, hipGetErrorString(e), file, line);
    set_error((int)e, buf);
    return (int)e;
}

struct Block { size_t size; hipStream_t last; bool idle; uint64_t freed_tick; hipEvent_t ev; bool ev_set; };
struct Pool {
    std::mutex mu;
    std::map<size_t, std::vector<void*>> free_lists;
    std::unordered_map<void*, Block> live;      // every block we own -> rounded size and last user
    size_t cached_bytes = 0, live_bytes = 0;
    hipEvent_t events[32] = {};
    unsigned next_event = 0;
    uint64_t tick = 0;                                                     // counts frees
    std::map<std::pair<hipStream_t, hipStream_t>, uint64_t> synced;        // (from, to) -> frees on `from` up to this tick are already waited for by `to`
};
static Pool& pool() { static Pool p; return p; }

static size_t round_size(size_t b) {
    if (b <= 256) return 256;
    if (b <= (size_t)1 << 20) {          // powers of two up to 1 MiB
        size_t s = 256;
        while (s < b) s <<= 1;
        return s;
    }
    const size_t g = (size_t)2 << 20;    // 2 MiB granules above
    return (b + g - 1) / g * g;
}

// The library's own streams and the default stream live as long as the process.  A caller's stream may be destroyed while
// blocks it used last still sit in the free lists, and a destroyed stream must never be passed to the runtime again: for
// such streams the event is recorded when the block is freed (the stream is certainly alive then) and kept with the block.
static std::mutex g_side_mu;
static hipStream_t g_side_streams[2][24] = {};
static bool is_persistent_stream(hipStream_t s) {
    if (s == nullptr) return true;
    std::lock_guard<std::mutex> lk(g_side_mu);
    for (auto& row : g_side_streams) for (hipStream_t t : row) if (t == s) return true;
    return false;
}

// Makes `stream` wait for what `blk`'s last user had queued when it let the block go.  Called with the pool locked.
static void order_behind_last_user(Pool& P, const Block& blk, hipStream_t stream) {
    if (blk.idle || blk.last == stream) return;
    if (blk.ev_set) {                                             // recorded at free time (any stream but the default one)
        if (hipStreamWaitEvent(stream, blk.ev, 0) != hipSuccess) { (void)hipGetLastError(); (void)hipDeviceSynchronize(); }
        return;
    }
    // What an earlier wait already covers is remembered only for takers that live as long as the process (the default stream and
    // the library's own): a caller's stream may be destroyed and its handle value given to a new stream, which has waited for
    // nothing.  A caller's stream gets its wait every time.
    uint64_t scratch_covered = 0;
    uint64_t& covered = is_persistent_stream(stream) ? P.synced[std::make_pair(blk.last, stream)] : scratch_covered;
    if (blk.freed_tick <= covered && covered != 0) return;      // an earlier wait of this stream on that one was placed after this block's free
    const uint64_t now = P.tick;
    hipEvent_t& ev = P.events[P.next_event++ % 32];
    if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); ev = nullptr; }
    // a wait takes the event's state at this call, so the event can be recorded again for the next block at once
    if (ev && hipEventRecord(ev, blk.last) == hipSuccess && hipStreamWaitEvent(stream, ev, 0) == hipSuccess) { covered = now; return; }
    (void)hipGetLastError();
    (void)hipDeviceSynchronize();        // no event: wait for everything
    covered = now;
}

void pool_note_wait(hipStream_t from, hipStream_t to) {
    if (from == to || !is_persistent_stream(from) || !is_persistent_stream(to)) return;
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    uint64_t& covered = P.synced[std::make_pair(from, to)];
    if (covered < P.tick) covered = P.tick;
}
// whether `stream` can take the block without another wait (called with the pool locked)
static bool needs_no_wait(Pool& P, const Block& b, hipStream_t stream) {
    if (b.idle || b.last == stream) return true;
    if (b.ev_set) return false;
    auto it = P.synced.find(std::make_pair(b.last, stream));
    return it != P.synced.end() && it->second != 0 && b.freed_tick <= it->second;
}

int pool_alloc(void** out, size_t bytes, hipStream_t stream, const hipStream_t* also) {
    Pool& P = pool();
    const size_t sz = round_size(bytes);
    {
        std::lock_guard<std::mutex> lk(P.mu);
        auto it = P.free_lists.find(sz);
        if (it != P.free_lists.end() && !it->second.empty()) {
            std::vector<void*>& fl = it->second;
            // prefer a block that needs no wait (same stream or idle) among the most recently freed
            size_t pick = fl.size() - 1;
            for (size_t k = 0; k < 8 && k < fl.size(); ++k) {
                const Block& b = P.live[fl[fl.size() - 1 - k]];
                if (needs_no_wait(P, b, stream)) { pick = fl.size() - 1 - k; break; }
            }
            void* p = fl[pick];
            fl[pick] = fl.back();
            fl.pop_back();
            order_behind_last_user(P, P.live[p], stream);
            if (also) order_behind_last_user(P, P.live[p], *also);
            P.cached_bytes -= sz;
            P.live_bytes += sz;
            *out = p;
            return 0;
        }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, sz);
    if (e != hipSuccess) {               // give cached blocks back and retry once
        (void)hipGetLastError();
        pool_trim();
        e = hipMalloc(&p, sz);
        if (e != hipSuccess) return hip_fail(e, "hipMalloc", __FILE__, __LINE__);
    }
    std::lock_guard<std::mutex> lk(P.mu);
    P.live[p] = Block{sz, stream, true, 0, nullptr, false};
    P.live_bytes += sz;
    *out = p;
    return 0;
}
int pool_free(void* p, hipStream_t stream, bool idle) {
    if (!p) return 0;
    const bool persistent = idle || is_persistent_stream(stream);
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    auto it = P.live.find(p);
    if (it == P.live.end()) { set_error(ZK_ERR_ARG, "zk_free: pointer was not allocated by zk_malloc"); return ZK_ERR_ARG; }
    Block& b = it->second;
    b.last = stream;
    b.idle = idle;
    b.freed_tick = ++P.tick;
    b.ev_set = false;
    // Any stream but the default one: the event is recorded now.  Recorded later, when another stream takes the block,
    // it would sit behind everything the freeing stream has been given since -- a whole opening or sumcheck job of the
    // library's own streams -- and the taker would wait for all of that, not for the block's last use.
    if (!idle && (!persistent || stream != nullptr)) {
        if (!b.ev && hipEventCreateWithFlags(&b.ev, hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); b.ev = nullptr; }
        if (b.ev && hipEventRecord(b.ev, stream) == hipSuccess) b.ev_set = true;
        else if (!persistent) { (void)hipGetLastError(); (void)hipStreamSynchronize(stream); b.idle = true; }
        else (void)hipGetLastError();      // a stream of the library's own: the wait is placed when the block is taken, as for the default stream
    }
    P.free_lists[it->second.size].push_back(p);
    P.cached_bytes += it->second.size;
    P.live_bytes -= it->second.size;
    return 0;
}
int pool_trim() {
    Pool& P = pool();
    std::vector<void*> victims;
    {
        std::lock_guard<std::mutex> lk(P.mu);
        for (auto& kv : P.free_lists) {
            for (void* p : kv.second) {
                victims.push_back(p);
                auto it = P.live.find(p);
                if (it != P.live.end()) { if (it->second.ev) (void)hipEventDestroy(it->second.ev); P.live.erase(it); }
            }
            kv.second.clear();
        }
        P.cached_bytes = 0;
    }
    if (!victims.empty()) (void)hipDeviceSynchronize();
    for (void* p : victims) (void)hipFree(p);
    return 0;
}

hipStream_t side_stream(int pool) {
    std::lock_guard<std::mutex> lk(g_side_mu);
    static unsigned next[2] = {0, 0};
    static int count[2] = {0, 0}, shared = 0;
    if (!count[0]) {
        count[0] = 8; count[1] = 2;       // an opening job takes two consecutive streams of pool 0 (folds / bucket sums); four jobs in flight
        if (const char* e = getenv("ZKLLM_SIDE_STREAMS")) {          // "openings,sumchecks[,shared]" (experiments)
            int a = 0, b2 = 0, c = 0;
            if (sscanf(e, "%d,%d,%d", &a, &b2, &c) >= 2 && a >= 1 && a <= 24 && b2 >= 1 && b2 <= 24) { count[0] = a; count[1] = b2; shared = c; }
        }
    }
    const int q = (pool && !shared) ? 1 : 0;
    const unsigned i = next[q]++ % (unsigned)count[q];
    hipStream_t& s = g_side_streams[q][i];
    // ZKLLM_SIDE_STREAMS_BLOCKING=1 (measurement only): streams that the default stream waits for and that wait for it; with
    // ZKLLM_SIDE_STREAMS=1,1,1 and a caller on the default stream no two kernels of the library overlap, so a kernel trace
    // shows what each costs alone
    static const bool blocking = [] { const char* e = getenv("ZKLLM_SIDE_STREAMS_BLOCKING"); return e && e[0] == '1'; }();
    if (!s && hipStreamCreateWithFlags(&s, blocking ? hipStreamDefault : hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); s = nullptr; return nullptr; }
    return s;
}

// hooks are registered by static initialisers of the other files: the list is made on first use and never destroyed
static std::mutex& shutdown_mu() { static std::mutex* m = new std::mutex; return *m; }
static std::vector<void (*)()>& shutdown_hooks() { static std::vector<void (*)()>* v = new std::vector<void (*)()>; return *v; }
void at_shutdown(void (*fn)()) { std::lock_guard<std::mutex> lk(shutdown_mu()); shutdown_hooks().push_back(fn); }

static std::mutex g_pinned_mu;
static std::vector<void*> g_pinned_free;
int pinned_acquire(void** host_ptr) {
    {
        std::lock_guard<std::mutex> lk(g_pinned_mu);
        if (!g_pinned_free.empty()) { *host_ptr = g_pinned_free.back(); g_pinned_free.pop_back(); return 0; }
    }
    void* p = nullptr;
    ZK_HIP(hipHostMalloc(&p, 64 << 10, hipHostMallocDefault));
    *host_ptr = p;
    return 0;
}
void pinned_release(void* host_ptr) {
    if (!host_ptr) return;
    std::lock_guard<std::mutex> lk(g_pinned_mu);
    g_pinned_free.push_back(host_ptr);
}

std::string last_error_text() { return g_err; }

namespace {
struct DeferBatch {
    void* pinned = nullptr;            // 64 KiB
    size_t used = 0;                   // field elements delivered so far
    std::vector<std::pair<size_t, int>> monts;      // (first element, count) to multiply by 2^256 on the way out
    hipEvent_t ev = nullptr;
    bool open = true;
};
thread_local DeferBatch* g_defer = nullptr;
}  // namespace
int deliver(hipStream_t st, const void* dev_src, void* host_dst, size_t count_fr, int n_mont) {
    using Fr = Big<8>;
    if (DeferBatch* b = g_defer) {
        ZK_ARG((b->used + count_fr) * sizeof(Fr) <= ((size_t)64 << 10), "deferred results: more than 64 KiB in one batch");
        ZK_HIP(hipMemcpyAsync((Fr*)b->pinned + b->used, dev_src, sizeof(Fr) * count_fr, hipMemcpyDeviceToHost, st));
        if (n_mont > 0) b->monts.emplace_back(b->used, n_mont);
        b->used += count_fr;
        return 0;
    }
    void* stage = nullptr;
    int rc = staging(&stage, sizeof(Fr) * count_fr);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, dev_src, sizeof(Fr) * count_fr, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    Fr* out = (Fr*)host_dst;
    memcpy(out, stage, sizeof(Fr) * count_fr);
    for (int i = 0; i < n_mont; ++i) out[i] = to_mont(out[i]);
    return 0;
}

namespace {
struct Launcher {
    std::mutex mu;
    std::condition_variable work, finished;
    std::deque<std::pair<uint64_t, std::pair<int, std::function<void()>>>> q;      // ticket, (device, closure)
    uint64_t next = 1, done = 0;
    bool stop = false, running = false;
    std::thread th;
    void loop() {
        int cur_dev = -1;
        std::unique_lock<std::mutex> lk(mu);
        for (;;) {
            work.wait(lk, [&] { return stop || !q.empty(); });
            if (q.empty()) return;      // stop, and nothing left
            auto item = std::move(q.front());
            q.pop_front();
            lk.unlock();
            if (item.second.first != cur_dev) { (void)hipSetDevice(item.second.first); cur_dev = item.second.first; }
            item.second.second();
            lk.lock();
            done = item.first;
            finished.notify_all();
        }
    }
};
Launcher& launcher() { static Launcher* L = new Launcher; return *L; }      // never destroyed: its thread may outlive static destruction
}  // namespace
static std::atomic<int> g_async_jobs{-1};      // -1: not decided yet (the environment decides at the first question)
bool launcher_enabled() {
    int v = g_async_jobs.load();
    if (v < 0) {
        const char* e = getenv("ZKLLM_ASYNC_JOBS");
        v = (e && e[0] == '0') ? 0 : 1;
        g_async_jobs.store(v);
    }
    return v != 0;
}
void launcher_set_enabled(bool on) { g_async_jobs.store(on ? 1 : 0); }
uint64_t launcher_submit(std::function<void()> fn) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    Launcher& L = launcher();
    std::lock_guard<std::mutex> lk(L.mu);
    if (!L.running) {
        L.stop = false;
        L.th = std::thread([&L] { L.loop(); });
        L.running = true;
    }
    const uint64_t t = L.next++;
    L.q.emplace_back(t, std::make_pair(dev, std::move(fn)));
    L.work.notify_one();
    return t;
}
void launcher_wait(uint64_t ticket) {
    if (!ticket) return;
    Launcher& L = launcher();
    std::unique_lock<std::mutex> lk(L.mu);
    L.finished.wait(lk, [&] { return L.done >= ticket; });
}
void launcher_stop() {
    Launcher& L = launcher();
    std::thread th;
    {
        std::lock_guard<std::mutex> lk(L.mu);
        if (!L.running) return;
        L.stop = true;
        L.work.notify_all();
        th = std::move(L.th);
        L.running = false;
    }
    th.join();          // the loop leaves once the queue is empty
}

int staging(void** host_ptr, size_t bytes) {
    static thread_local void* buf = nullptr;     // one per host thread, kept until the process ends
    static const size_t cap = 64 << 10;
    ZK_ARG(bytes <= cap, "staging request over 64 KiB");
    if (!buf) ZK_HIP(hipHostMalloc(&buf, cap, hipHostMallocDefault));
    *host_ptr = buf;
    return 0;
}

}  // namespace zk

using namespace zk;

extern "C" {

const char* zk_last_error(void) { return g_err.c_str(); }

int zk_init(int device) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        set_error(ZK_ERR_NO_DEVICE, "no HIP device visible");
        return ZK_ERR_NO_DEVICE;
    }
    ZK_ARG(device >= 0 && device < n, "zk_init: device index out of range");
    ZK_HIP(hipSetDevice(device));
    return fr_static_scratch_setup();     // zk_fr_sum_static's array: its address on this device, looked up once
}
int zk_device_info(char* name, int name_len, int* compute_units, int* clock_khz, size_t* total_mem) {
    hipDeviceProp_t prop;
    int dev = 0;
    ZK_HIP(hipGetDevice(&dev));
    ZK_HIP(hipGetDeviceProperties(&prop, dev));
    if (name && name_len > 0) { strncpy(name, prop.gcnArchName, name_len - 1); name[name_len - 1] = 0; }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return 0;
}
int zk_malloc(void** out, size_t bytes) { ZK_ARG(out != nullptr, "zk_malloc: null out"); return pool_alloc(out, bytes ? bytes : 1, nullptr); }
int zk_free(void* p) { return pool_free(p, nullptr); }
int zk_free_async(void* p, void* stream) { return pool_free(p, (hipStream_t)stream); }
int zk_pool_trim(void) { return pool_trim(); }
// Releases what the library holds on the device and in the runtime, in a fixed order, while the runtime is certainly alive:
// waits for the device, lets the kernel files drop their timing events, gives the cached blocks back (live blocks stay with
// their owners), destroys the library's streams and the allocator's events and frees the pinned buffers that are not in use.
// The library stays usable: streams and buffers are made again on demand.  For a host that wants nothing of this left to
// static destruction at process exit.
int zk_shutdown(void) {
    launcher_stop();          // whatever was handed to the launch thread is on its streams before the device is waited for
    (void)hipDeviceSynchronize();
    {
        std::lock_guard<std::mutex> lk(shutdown_mu());
        for (void (*fn)() : shutdown_hooks()) fn();
    }
    pool_trim();
    {
        std::lock_guard<std::mutex> lk(g_side_mu);
        for (auto& row : g_side_streams)
            for (hipStream_t& t : row)
                if (t) { (void)hipStreamDestroy(t); t = nullptr; }
    }
    {
        Pool& P = pool();
        std::lock_guard<std::mutex> lk(P.mu);
        for (hipEvent_t& e : P.events) if (e) { (void)hipEventDestroy(e); e = nullptr; }
        P.synced.clear();
        for (auto& kv : P.live) if (kv.second.ev) { (void)hipEventDestroy(kv.second.ev); kv.second.ev = nullptr; kv.second.ev_set = false; kv.second.idle = true; }      // the device is idle
    }
    {
        std::lock_guard<std::mutex> lk(g_pinned_mu);
        for (void* p : g_pinned_free) (void)hipHostFree(p);
        g_pinned_free.clear();
    }
    (void)hipGetLastError();
    return 0;
}
int zk_defer_begin(void** batch) {
    ZK_ARG(batch != nullptr, "zk_defer_begin: null argument");
    ZK_ARG(g_defer == nullptr, "zk_defer_begin: this thread already has a batch open");
    DeferBatch* b = new DeferBatch;
    int rc = pinned_acquire(&b->pinned);
    if (rc) { delete b; return rc; }
    g_defer = b;
    *batch = b;
    return 0;
}
int zk_defer_end(void* batch, void* stream) {
    DeferBatch* b = (DeferBatch*)batch;
    ZK_ARG(b != nullptr && b == g_defer && b->open, "zk_defer_end: not this thread's open batch");
    g_defer = nullptr;
    b->open = false;
    ZK_HIP(hipEventCreateWithFlags(&b->ev, hipEventDisableTiming));
    ZK_HIP(hipEventRecord(b->ev, (hipStream_t)stream));
    return 0;
}
int zk_defer_wait(void* batch, uint32_t* out_host, size_t max_fr, size_t* n_fr) {
    using Fr = Big<8>;
    DeferBatch* b = (DeferBatch*)batch;
    ZK_ARG(b != nullptr && !b->open && b->ev != nullptr, "zk_defer_wait: the batch has not been ended");
    ZK_ARG(b->used <= max_fr, "zk_defer_wait: more results than the buffer holds");
    ZK_HIP(hipEventSynchronize(b->ev));
    Fr* out = (Fr*)out_host;
    memcpy(out, b->pinned, sizeof(Fr) * b->used);
    for (auto& m : b->monts)
        for (int i = 0; i < m.second; ++i) out[m.first + i] = to_mont(out[m.first + i]);
    if (n_fr) *n_fr = b->used;
    return 0;
}
int zk_defer_free(void* batch) {
    DeferBatch* b = (DeferBatch*)batch;
    if (!b) return 0;
    if (b == g_defer) g_defer = nullptr;
    if (b->ev) { (void)hipEventSynchronize(b->ev); (void)hipEventDestroy(b->ev); }      // the copies into the pinned buffer have landed
    else if (b->used) (void)hipDeviceSynchronize();                                   // never ended: wait for whatever was queued
    pinned_release(b->pinned);
    delete b;
    return 0;
}
int zk_set_async_jobs(int on) { launcher_set_enabled(on != 0); return 0; }
int zk_async_jobs(void) { return launcher_enabled() ? 1 : 0; }
int zk_pool_stats(size_t* live_bytes, size_t* cached_bytes) {
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    if (live_bytes) *live_bytes = P.live_bytes;
    if (cached_bytes) *cached_bytes = P.cached_bytes;
    return 0;
}
int zk_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return 0;
    ZK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    ZK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
int zk_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return 0;
    ZK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    ZK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
int zk_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return 0;
    ZK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}
int zk_memset(void* dst, int value, size_t bytes, void* stream) {
    if (!bytes) return 0;
    ZK_HIP(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
    return 0;
}
int zk_sync(void* stream) {
    ZK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
int zk_event_create(void** ev) { hipEvent_t e; ZK_HIP(hipEventCreate(&e)); *ev = (void*)e; return 0; }
int zk_event_destroy(void* ev) { ZK_HIP(hipEventDestroy((hipEvent_t)ev)); return 0; }
int zk_event_record(void* ev, void* stream) { ZK_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream)); return 0; }
int zk_event_elapsed_ms(void* start, void* stop, float* ms) {
    ZK_HIP(hipEventSynchronize((hipEvent_t)stop));
    ZK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

}  // extern "C"

// Runtime pieces of the C ABI: device selection, the caching allocator, copies, error text.
#include <cstdlib>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>
#include <cstdio>
#include <cstring>
#include "rt.hpp"
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

struct Pool {
    std::mutex mu;
    std::map<size_t, std::vector<void*>> free_lists;
    std::unordered_map<void*, size_t> live;     // every block we own -> rounded size
    size_t cached_bytes = 0, live_bytes = 0;
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

int pool_alloc(void** out, size_t bytes) {
    Pool& P = pool();
    const size_t sz = round_size(bytes);
    {
        std::lock_guard<std::mutex> lk(P.mu);
        auto it = P.free_lists.find(sz);
        if (it != P.free_lists.end() && !it->second.empty()) {
            *out = it->second.back();
            it->second.pop_back();
            P.cached_bytes -= sz;
            P.live_bytes += sz;
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
    P.live[p] = sz;
    P.live_bytes += sz;
    *out = p;
    return 0;
}
int pool_free(void* p) {
    if (!p) return 0;
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    auto it = P.live.find(p);
    if (it == P.live.end()) { set_error(ZK_ERR_ARG, "zk_free: pointer was not allocated by zk_malloc"); return ZK_ERR_ARG; }
    P.free_lists[it->second].push_back(p);
    P.cached_bytes += it->second;
    P.live_bytes -= it->second;
    return 0;
}
int pool_trim() {
    Pool& P = pool();
    std::vector<void*> victims;
    {
        std::lock_guard<std::mutex> lk(P.mu);
        for (auto& kv : P.free_lists) {
            for (void* p : kv.second) { victims.push_back(p); P.live.erase(p); }
            kv.second.clear();
        }
        P.cached_bytes = 0;
    }
    if (!victims.empty()) (void)hipDeviceSynchronize();
    for (void* p : victims) (void)hipFree(p);
    return 0;
}

hipStream_t side_stream(int pool) {
    static hipStream_t streams[2][8] = {};
    static unsigned next[2] = {0, 0};
    static int count[2] = {0, 0}, shared = 0;
    if (!count[0]) {
        count[0] = 6; count[1] = 2;       // an opening takes two consecutive streams of pool 0 (folds / bucket sums); three openings in flight
        if (const char* e = getenv("ZKLLM_SIDE_STREAMS")) {          // "openings,sumchecks[,shared]" (experiments)
            int a = 0, b2 = 0, c = 0;
            if (sscanf(e, "%d,%d,%d", &a, &b2, &c) >= 2 && a >= 1 && a <= 8 && b2 >= 1 && b2 <= 8) { count[0] = a; count[1] = b2; shared = c; }
        }
    }
    const int q = (pool && !shared) ? 1 : 0;
    const unsigned i = next[q]++ % (unsigned)count[q];
    if (!streams[q][i] && hipStreamCreateWithFlags(&streams[q][i], hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); streams[q][i] = nullptr; return nullptr; }
    return streams[q][i];
}

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

int staging(void** host_ptr, size_t bytes) {
    static void* buf = nullptr;
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
int zk_malloc(void** out, size_t bytes) { ZK_ARG(out != nullptr, "zk_malloc: null out"); return pool_alloc(out, bytes ? bytes : 1); }
int zk_free(void* p) { return pool_free(p); }
int zk_pool_trim(void) { return pool_trim(); }
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

#include <memory>
#include "fr-tensor.hpp"
#include <chrono>

#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <random>

#include "../../include/zkllm_hip.h"
#include "../csrc/field.hpp"
#include "ioutils.hpp"

using namespace std;

// ---- status / globals ---------------------------------------------------------------------------
void zk_check(int rc, const char* where) {
    if (rc != 0) throw std::runtime_error(string(where) + ": " + zk_last_error());
}
#define ZKC(call) zk_check((call), #call)

namespace {
struct Globals {
    std::mt19937 mt;
    bool seeded = false;
    int matmul_mode = 0;
    int last_matmul_path = 0;
    bool recording = false;
    std::vector<Fr_t> transcript;
    std::vector<G1Jacobian_t> transcript_g1;
    std::string proof_file;
    unsigned long long drawn = 0;                                             // challenge elements drawn so far
    std::deque<std::pair<unsigned long long, std::vector<Fr_t>>> draw_log;    // recent short draws with their positions
    Globals() {
        if (const char* m = getenv("ZKLLM_MATMUL")) matmul_mode = (string(m) == "generic") ? 1 : 0;
        if (const char* f = getenv("ZKLLM_PROOF_FILE")) { proof_file = f; recording = !proof_file.empty(); }
    }
    ~Globals() {
        if (!proof_file.empty()) try { zk_write_proof_file(proof_file); } catch (...) {}
    }
};
Globals& G() { static Globals g; return g; }
void ensure_seeded() {
    Globals& g = G();
    if (g.seeded) return;
    if (const char* s = getenv("ZKLLM_SEED")) g.mt.seed((uint32_t)strtoul(s, nullptr, 10));
    else { std::random_device rd; g.mt.seed(rd()); }
    g.seeded = true;
}
}  // namespace

void zk_seed_challenges(uint32_t seed) { G().mt.seed(seed); G().seeded = true; G().drawn = 0; G().draw_log.clear(); }
void zk_set_matmul_mode(int mode) { G().matmul_mode = mode; }
int zk_last_matmul_path() { return G().last_matmul_path; }
void zk_transcript_begin() { G().transcript.clear(); G().transcript_g1.clear(); G().recording = true; }
void zk_record_g1(const std::vector<G1Jacobian_t>& points) { if (G().recording) G().transcript_g1.insert(G().transcript_g1.end(), points.begin(), points.end()); }
const std::vector<G1Jacobian_t>& zk_transcript_g1() { return G().transcript_g1; }
void zk_write_proof_file(const std::string& path) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) throw std::runtime_error("zk_write_proof_file: cannot open " + path);
    const Globals& g = G();
    const uint64_t counts[2] = {(uint64_t)g.transcript.size(), (uint64_t)g.transcript_g1.size()};
    bool ok = fwrite("ZKLLMPF1", 1, 8, f) == 8 && fwrite(counts, 8, 2, f) == 2;
    if (ok && counts[0]) ok = fwrite(g.transcript.data(), sizeof(Fr_t), counts[0], f) == counts[0];
    if (ok && counts[1]) ok = fwrite(g.transcript_g1.data(), sizeof(G1Jacobian_t), counts[1], f) == counts[1];
    fclose(f);
    if (!ok) throw std::runtime_error("zk_write_proof_file: short write to " + path);
}
const std::vector<Fr_t>& zk_transcript() { return G().transcript; }
void zk_transcript_end() { G().recording = false; }
// entries go to `sink` instead while one is set (a block whose proof is collected out of turn); zk_record_insert puts them in place
static std::vector<Fr_t>* g_record_sink = nullptr;
void zk_record_divert(std::vector<Fr_t>* sink) { g_record_sink = sink; }
void zk_record_insert(size_t pos, const std::vector<Fr_t>& xs) {
    if (!G().recording || xs.empty()) return;
    auto& t = G().transcript;
    t.insert(t.begin() + (pos < t.size() ? pos : t.size()), xs.begin(), xs.end());
}
void zk_record(const Fr_t& x) { if (G().recording) (g_record_sink ? *g_record_sink : G().transcript).push_back(x); }
namespace {
struct PhaseTimes {
    bool on = false;
    std::chrono::steady_clock::time_point last;
    std::vector<std::pair<std::string, double>> ms;
};
PhaseTimes& phases() { static PhaseTimes p; return p; }
}  // namespace
void zk_phase_end(const char* name) {
    PhaseTimes& p = phases();
    if (!p.on) return;
    (void)zk_sync(nullptr);
    const auto now = std::chrono::steady_clock::now();
    const double d = std::chrono::duration<double, std::milli>(now - p.last).count();
    p.last = now;
    for (auto& kv : p.ms) if (kv.first == name) { kv.second += d; return; }
    p.ms.emplace_back(name, d);
}
ZkLibraryScope::ZkLibraryScope() {
    const char* e = getenv("ZKLLM_TIMING");
    phases().on = e && e[0] == '1';
    phases().last = std::chrono::steady_clock::now();
}
ZkLibraryScope::~ZkLibraryScope() {
    zk_phase_end("release_ms");
    (void)zk_shutdown();
    PhaseTimes& p = phases();
    if (p.on) {
        zk_phase_end("shutdown_ms");
        std::cerr << "ZKLLM_TIMES {";
        for (size_t i = 0; i < p.ms.size(); ++i) std::cerr << (i ? ", " : "") << "\"" << p.ms[i].first << "\": " << p.ms[i].second;
        std::cerr << "}" << std::endl;
    }
}
size_t zk_record_reserve() {
    if (!G().recording) return (size_t)-1;
    if (g_record_sink) throw std::runtime_error("zk_record_reserve: no position can be reserved while the entries are diverted");
    G().transcript.push_back(Fr_t{{0, 0, 0, 0, 0, 0, 0, 0}});
    return G().transcript.size() - 1;
}
void zk_record_fill(size_t slot, const Fr_t& x) { if (slot != (size_t)-1 && slot < G().transcript.size()) G().transcript[slot] = x; }
void zk_record(const std::vector<Fr_t>& xs) {
    if (!G().recording) return;
    auto& t = g_record_sink ? *g_record_sink : G().transcript;
    t.insert(t.end(), xs.begin(), xs.end());
}

ostream& operator<<(ostream& os, const Fr_t& x) {
    os << "0x" << std::hex;
    for (uint i = 8; i > 0; --i) os << std::setfill('0') << std::setw(8) << x.val[i - 1];
    return os << std::dec << std::setw(0) << std::setfill(' ');
}

// 8 raw mt19937 outputs per element, the last reduced mod the top limb of r (fr-tensor.cu:16-24)
static void draw_elements(std::mt19937& mt, vector<Fr_t>& out) {
    for (size_t i = 0; i < out.size(); ++i) {
        for (int k = 0; k < 7; ++k) out[i].val[k] = (uint)mt();
        out[i].val[7] = (uint)mt() % 1944954707u;
    }
}
vector<Fr_t> random_vec(uint len) {
    ensure_seeded();
    Globals& g = G();
    vector<Fr_t> out(len);
    draw_elements(g.mt, out);
    if (len >= 1 && len <= 64) {
        g.draw_log.emplace_back(g.drawn, out);
        if (g.draw_log.size() > 4096) g.draw_log.pop_front();
    }
    g.drawn += len;
    return out;
}
unsigned long long zk_challenge_position() { return G().drawn; }
vector<Fr_t> zk_challenge_peek(unsigned long long ahead, uint len) {
    ensure_seeded();
    std::mt19937 mt = G().mt;          // a copy: the stream itself does not move
    mt.discard(8ull * ahead);
    vector<Fr_t> out(len);
    draw_elements(mt, out);
    return out;
}
bool zk_challenge_find(const vector<Fr_t>& v, unsigned long long* position) {
    if (v.empty()) { *position = G().drawn; return true; }          // an empty draw sits anywhere
    const auto& log = G().draw_log;
    for (auto it = log.rbegin(); it != log.rend(); ++it)
        if (it->second.size() == v.size() && std::memcmp(it->second.data(), v.data(), v.size() * sizeof(Fr_t)) == 0) { *position = it->first; return true; }
    return false;
}

uint ceilLog2(uint num) {
    if (num == 0) return 0;
    num--;
    uint result = 0;
    while (num > 0) { num >>= 1; result++; }
    return result;
}

// ---- raw device buffers / files -----------------------------------------------------------------------
DevBuf::DevBuf(size_t bytes) { ZKC(zk_malloc(&p, bytes)); }
DevBuf::~DevBuf() { if (p) zk_free(p); }

void savebin(const string& filename, const void* gpudata, size_t size) {
    std::vector<char> data(size);
    ZKC(zk_memcpy_d2h(data.data(), gpudata, size, nullptr));
    FILE* f = fopen(filename.c_str(), "wb");
    if (!f) throw std::runtime_error("savebin: cannot open " + filename);
    size_t w = fwrite(data.data(), 1, size, f);
    fclose(f);
    if (w != size) throw std::runtime_error("savebin: short write to " + filename);
}
size_t findsize(const string& filename) {
    FILE* f = fopen(filename.c_str(), "rb");
    if (!f) throw std::runtime_error("findsize: cannot open " + filename);
    fseek(f, 0, SEEK_END);
    long sz = ftell(f);
    fclose(f);
    return (size_t)sz;
}
void loadbin(const string& filename, void* gpudata, size_t size) {
    std::vector<char> data(size);
    FILE* f = fopen(filename.c_str(), "rb");
    if (!f) throw std::runtime_error("loadbin: cannot open " + filename);
    size_t r = fread(data.data(), 1, size, f);
    fclose(f);
    if (r != size) throw std::runtime_error("loadbin: short read from " + filename);
    ZKC(zk_memcpy_h2d(gpudata, data.data(), size, nullptr));
}

// ---- FrTensor -------------------------------------------------------------------------------------------
static Fr_t* fr_alloc(size_t n) {
    void* p = nullptr;
    ZKC(zk_malloc(&p, sizeof(Fr_t) * (n ? n : 1)));
    return (Fr_t*)p;
}

FrTensor::FrTensor(uint size) : gpu_data(fr_alloc(size)), size(size) {}
FrTensor::FrTensor(uint size, const Fr_t* cpu_data) : gpu_data(fr_alloc(size)), size(size) {
    ZKC(zk_memcpy_h2d(gpu_data, cpu_data, sizeof(Fr_t) * size, nullptr));
}
FrTensor::FrTensor(uint size, const int* cpu_data) : gpu_data(fr_alloc(size)), size(size) {
    DevBuf tmp(sizeof(int) * (size_t)size);
    ZKC(zk_memcpy_h2d(tmp.p, cpu_data, sizeof(int) * (size_t)size, nullptr));
    ZKC(zk_fr_from_i32(gpu_data, tmp.p, size, nullptr));
    ZKC(zk_sync(nullptr));
}
FrTensor::FrTensor(uint size, const long* cpu_data) : gpu_data(fr_alloc(size)), size(size) {
    DevBuf tmp(sizeof(long) * (size_t)size);
    ZKC(zk_memcpy_h2d(tmp.p, cpu_data, sizeof(long) * (size_t)size, nullptr));
    ZKC(zk_fr_from_i64(gpu_data, tmp.p, size, nullptr));
    ZKC(zk_sync(nullptr));
}
FrTensor::FrTensor(uint size, const float* cpu_data, unsigned long sf) : gpu_data(fr_alloc(size)), size(size) {
    DevBuf tmp(sizeof(float) * (size_t)size);
    ZKC(zk_memcpy_h2d(tmp.p, cpu_data, sizeof(float) * (size_t)size, nullptr));
    ZKC(zk_fr_from_f32(gpu_data, tmp.p, sf, size, nullptr));
    ZKC(zk_sync(nullptr));
}
FrTensor::FrTensor(uint size, const double* cpu_data, unsigned long sf) : gpu_data(fr_alloc(size)), size(size) {
    DevBuf tmp(sizeof(double) * (size_t)size);
    ZKC(zk_memcpy_h2d(tmp.p, cpu_data, sizeof(double) * (size_t)size, nullptr));
    ZKC(zk_fr_from_f64(gpu_data, tmp.p, sf, size, nullptr));
    ZKC(zk_sync(nullptr));
}
FrTensor::FrTensor(const FrTensor& t) : gpu_data(fr_alloc(t.size)), size(t.size) {
    ZKC(zk_memcpy_d2d(gpu_data, t.gpu_data, sizeof(Fr_t) * (size_t)size, nullptr));
}
FrTensor::FrTensor(FrTensor&& t) noexcept
    : gpu_data(t.gpu_data), size(t.size), borrowed(t.borrowed), rhs_cache(std::move(t.rhs_cache)), fold_cache(std::move(t.fold_cache)) { t.gpu_data = nullptr; }
void MatmulRhsCache::reset() {
    if (prepared) zk_fr_matmul_rhs_free(prepared);
    prepared = nullptr;
}
FrTensor::FrTensor(const FrTensor& t, ViewTag) : gpu_data(t.gpu_data), size(t.size), borrowed(true), rhs_cache(t.rhs_cache), fold_cache(t.fold_cache) {}
FrTensor FrTensor::view(const FrTensor& t) { return FrTensor(t, ViewTag{}); }
void FrTensor::keep_as_matmul_rhs() {
    if (!rhs_cache) rhs_cache = std::make_shared<MatmulRhsCache>();
}
void FoldCache::reset() {
    if (prepared) zk_fr_fold_prepared_free(prepared);
    prepared = nullptr;
    tried = false;
    if (unchecked) zk_free(unchecked);
    unchecked = nullptr;
}
void FoldCache::settle() {
    if (!unchecked) return;
    uint32_t bad = 0;
    const int rc = zk_memcpy_d2h(&bad, unchecked, 4, nullptr);          // waits for the producing kernel
    zk_free(unchecked);
    unchecked = nullptr;
    if (rc || bad) {
        if (prepared) zk_fr_fold_prepared_free(prepared);
        prepared = nullptr;          // tried stays set: the elements are known not to be 32-bit integers
    }
    zk_check(rc, "zk_memcpy_d2h");
}
void* FrTensor::ints_for_producer_unchecked(void** bad_flag_dev) {
    void* ints = ints_for_producer();
    ZKC(zk_malloc(&fold_cache->unchecked, 4));
    *bad_flag_dev = fold_cache->unchecked;
    return ints;
}
void FrTensor::keep_for_folds() {
    if (!fold_cache) fold_cache = std::make_shared<FoldCache>();
    if (!fold_cache->tried) {
        fold_cache->tried = true;
        ZKC(zk_fr_fold_prepare(&fold_cache->prepared, gpu_data, size, nullptr));
    }
}
void* FrTensor::ints_for_producer() {
    if (!fold_cache) fold_cache = std::make_shared<FoldCache>();
    fold_cache->reset();
    void* ints = nullptr;
    ZKC(zk_fr_fold_prepared_new(&fold_cache->prepared, &ints, size, nullptr));
    fold_cache->tried = true;
    return ints;
}
void FrTensor::drop_kept() {
    if (rhs_cache) rhs_cache->reset();
    if (fold_cache) fold_cache->reset();
}
FrTensor::FrTensor(const string& filename) : gpu_data(nullptr), size((uint)(findsize(filename) / sizeof(Fr_t))) {
    gpu_data = fr_alloc(size);
    loadbin(filename, gpu_data, sizeof(Fr_t) * (size_t)size);
}
FrTensor::~FrTensor() {
    if (gpu_data && !borrowed) zk_free(gpu_data);
    gpu_data = nullptr;
}

FrTensor FrTensor::from_int_bin(const string& filename) {
    size_t n = findsize(filename) / sizeof(int);
    FrTensor out((uint)n);
    DevBuf tmp(sizeof(int) * n);
    loadbin(filename, tmp.p, sizeof(int) * n);
    ZKC(zk_fr_from_i32(out.gpu_data, tmp.p, n, nullptr));
    ZKC(zk_sync(nullptr));
    return out;
}
// The reference loads only sizeof(int)*size bytes here (fr-tensor.cu:243-244); this reads all of them.
FrTensor FrTensor::from_long_bin(const string& filename) {
    size_t n = findsize(filename) / sizeof(long);
    FrTensor out((uint)n);
    DevBuf tmp(sizeof(long) * n);
    loadbin(filename, tmp.p, sizeof(long) * n);
    ZKC(zk_fr_from_i64(out.gpu_data, tmp.p, n, nullptr));
    ZKC(zk_sync(nullptr));
    return out;
}
void FrTensor::save(const string& filename) const { savebin(filename, gpu_data, sizeof(Fr_t) * (size_t)size); }
void FrTensor::save_int(const string& filename) const {
    DevBuf tmp(sizeof(int) * (size_t)size);
    ZKC(zk_fr_to_i32(tmp.p, gpu_data, size, nullptr));
    savebin(filename, tmp.p, sizeof(int) * (size_t)size);
}
void FrTensor::save_long(const string& filename) const {
    DevBuf tmp(sizeof(long) * (size_t)size);
    ZKC(zk_fr_to_i64(tmp.p, gpu_data, size, nullptr));
    savebin(filename, tmp.p, sizeof(long) * (size_t)size);
}

Fr_t FrTensor::operator()(uint idx) const {
    if (idx >= size) throw std::runtime_error("FrTensor::operator(): index out of range");
    Fr_t out;
    ZKC(zk_memcpy_d2h(&out, gpu_data + idx, sizeof(Fr_t), nullptr));
    return out;
}

#define SAME_SIZE(t) if (size != (t).size) throw std::runtime_error("Incompatible dimensions")

FrTensor FrTensor::operator+(const FrTensor& t) const { SAME_SIZE(t); FrTensor out(size); ZKC(zk_fr_add(out.gpu_data, gpu_data, t.gpu_data, size, nullptr)); return out; }
FrTensor FrTensor::operator+(const Fr_t& x) const { FrTensor out(size); ZKC(zk_fr_add_s(out.gpu_data, gpu_data, x.val, size, nullptr)); return out; }
FrTensor& FrTensor::operator+=(const FrTensor& t) { SAME_SIZE(t); drop_kept(); ZKC(zk_fr_add(gpu_data, gpu_data, t.gpu_data, size, nullptr)); return *this; }
FrTensor& FrTensor::operator+=(const Fr_t& x) { drop_kept(); ZKC(zk_fr_add_s(gpu_data, gpu_data, x.val, size, nullptr)); return *this; }
FrTensor FrTensor::operator-() const { FrTensor out(size); ZKC(zk_fr_neg(out.gpu_data, gpu_data, size, nullptr)); return out; }
FrTensor FrTensor::operator-(const FrTensor& t) const { SAME_SIZE(t); FrTensor out(size); ZKC(zk_fr_sub(out.gpu_data, gpu_data, t.gpu_data, size, nullptr)); return out; }
FrTensor FrTensor::operator-(const Fr_t& x) const { FrTensor out(size); ZKC(zk_fr_sub_s(out.gpu_data, gpu_data, x.val, size, nullptr)); return out; }
FrTensor& FrTensor::operator-=(const FrTensor& t) { SAME_SIZE(t); drop_kept(); ZKC(zk_fr_sub(gpu_data, gpu_data, t.gpu_data, size, nullptr)); return *this; }
FrTensor& FrTensor::operator-=(const Fr_t& x) { drop_kept(); ZKC(zk_fr_sub_s(gpu_data, gpu_data, x.val, size, nullptr)); return *this; }
FrTensor& FrTensor::mont() { drop_kept(); ZKC(zk_fr_mont(gpu_data, gpu_data, size, nullptr)); return *this; }
FrTensor& FrTensor::unmont() { drop_kept(); ZKC(zk_fr_unmont(gpu_data, gpu_data, size, nullptr)); return *this; }
FrTensor FrTensor::operator*(const FrTensor& t) const {
    SAME_SIZE(t);
    FrTensor out(size);
    if (kept_ints() && t.kept_ints()) ZKC(zk_fr_mul_ints(out.gpu_data, kept_ints(), t.kept_ints(), size, nullptr));      // exact 64-bit products
    else ZKC(zk_fr_mul(out.gpu_data, gpu_data, t.gpu_data, size, nullptr));
    return out;
}
FrTensor FrTensor::operator*(const Fr_t& x) const { FrTensor out(size); ZKC(zk_fr_mul_s(out.gpu_data, gpu_data, x.val, size, nullptr)); return out; }
FrTensor& FrTensor::operator*=(const FrTensor& t) { SAME_SIZE(t); drop_kept(); ZKC(zk_fr_mul(gpu_data, gpu_data, t.gpu_data, size, nullptr)); return *this; }
FrTensor& FrTensor::operator*=(const Fr_t& x) { drop_kept(); ZKC(zk_fr_mul_s(gpu_data, gpu_data, x.val, size, nullptr)); return *this; }
FrTensor& FrTensor::operator=(const FrTensor& t) {
    if (size != t.size) throw std::runtime_error("operator=: Incompatible dimensions");
    drop_kept();
    ZKC(zk_memcpy_d2d(gpu_data, t.gpu_data, sizeof(Fr_t) * (size_t)size, nullptr));
    return *this;
}

Fr_t FrTensor::sum() const {
    Fr_t out;
    ZKC(zk_fr_sum(out.val, gpu_data, size, nullptr));
    return out;
}

Fr_t FrTensor::operator()(const vector<Fr_t>& u) const {
    uint log_dim = (uint)u.size();
    if (size <= ((1u << log_dim) / 2) || size > (1u << log_dim)) throw std::runtime_error("Incompatible dimensions");
    Fr_t out;
    if (const void* h = kept_ints()) {          // read from the int32 form
        const void* x = gpu_data;
        ZKC(zk_fr_me_multi_ints(out.val, &x, &h, 1, size, u.empty() ? nullptr : u[0].val, (int)log_dim, nullptr));
        return out;
    }
    ZKC(zk_fr_me(out.val, gpu_data, size, u.empty() ? nullptr : u[0].val, (int)log_dim, nullptr));
    return out;
}

DeferredResults& DeferredResults::operator=(DeferredResults&& o) noexcept {
    if (this != &o) {
        if (batch) zk_defer_free(batch);
        batch = o.batch; open = o.open;
        o.batch = nullptr; o.open = false;
    }
    return *this;
}
DeferredResults::~DeferredResults() { if (batch) zk_defer_free(batch); }
void DeferredResults::begin() {
    if (batch) throw std::runtime_error("DeferredResults::begin: already begun");
    ZKC(zk_defer_begin(&batch));
    open = true;
}
void DeferredResults::end() {
    if (!batch || !open) throw std::runtime_error("DeferredResults::end: nothing open");
    open = false;
    ZKC(zk_defer_end(batch, nullptr));
}
std::vector<Fr_t> DeferredResults::wait() {
    if (!batch || open) throw std::runtime_error("DeferredResults::wait: not ended");
    std::vector<Fr_t> out(2048);
    size_t n = 0;
    const int rc = zk_defer_wait(batch, out[0].val, out.size(), &n);
    zk_defer_free(batch);
    batch = nullptr;
    zk_check(rc, "zk_defer_wait");
    out.resize(n);
    return out;
}

vector<Fr_t> FrTensor::me_batch(const vector<const FrTensor*>& ts, const vector<Fr_t>& u) {
    vector<Fr_t> out(ts.size());
    if (ts.empty()) return out;
    const uint log_dim = (uint)u.size();
    const uint n = ts[0]->size;
    if (n <= ((1u << log_dim) / 2) || n > (1u << log_dim)) throw std::runtime_error("Incompatible dimensions");
    for (auto* t : ts) if (t->size != n) throw std::runtime_error("me_batch: tensors of different sizes");
    for (size_t i0 = 0; i0 < ts.size(); i0 += 8) {
        const int K = (int)std::min<size_t>(8, ts.size() - i0);
        const void *ptrs[8], *ints[8];
        bool any = false;
        for (int i = 0; i < K; ++i) { ptrs[i] = ts[i0 + i]->gpu_data; ints[i] = ts[i0 + i]->kept_ints(); any = any || ints[i]; }
        if (any) ZKC(zk_fr_me_multi_ints(out[i0].val, ptrs, ints, K, n, u.empty() ? nullptr : u[0].val, (int)log_dim, nullptr));
        else ZKC(zk_fr_me_multi(out[i0].val, ptrs, K, n, u.empty() ? nullptr : u[0].val, (int)log_dim, nullptr));
    }
    return out;
}

// Folds `u.size()` levels of the middle axis, up to three levels per pass.
static FrTensor fold_axis_all(const FrTensor& t, const vector<Fr_t>& u, uint cur_dim, size_t window) {
    if (u.empty()) return t;
    if ((size_t)t.size % ((size_t)cur_dim * window) != 0) throw std::runtime_error("t.size % (cur_dim * window_size) != 0");
    const size_t other = (size_t)t.size / ((size_t)cur_dim * window);
    if (FoldCache* fc = t.fold_cache.get(); fc && u.size() <= 24 && cur_dim <= (1u << u.size())) {
        if (fc->unchecked) fc->settle();
        if (!fc->tried) {
            fc->tried = true;
            ZKC(zk_fr_fold_prepare(&fc->prepared, t.gpu_data, t.size, nullptr));
        }
        if (fc->prepared) {
            FrTensor out((uint)(other * window));
            ZKC(zk_fr_fold_axis_prepared(out.gpu_data, fc->prepared, u[0].val, (int)u.size(), other, cur_dim, window, nullptr));
            return out;
        }
    }
    const Fr_t* src = t.gpu_data;
    std::vector<FrTensor> keep;   // intermediates stay alive until the last pass has been queued
    size_t done = 0;
    uint cur = cur_dim;
    while (done < u.size()) {
        const int L = (int)std::min<size_t>(3, u.size() - done);
        const uint cur_out = (uint)(((uint64_t)cur + (1u << L) - 1) >> L);
        keep.emplace_back((uint)(other * cur_out * window));
        ZKC(zk_fr_fold_axis(keep.back().gpu_data, src, u[done].val, L, other, cur, window, nullptr));
        src = keep.back().gpu_data;
        cur = cur_out;
        done += L;
    }
    FrTensor out(std::move(keep.back()));
    return out;
}

// Deprecated window fold (fr-tensor.cu:512-516, :612-641): adjacent windows of the flat tensor,
// zero-extended to a whole number of window pairs at every level.
FrTensor FrTensor::partial_me(const vector<Fr_t>& u, uint window_size) const {
    if (u.empty()) return *this;
    if (size <= window_size * (1u << (u.size() - 1))) throw std::runtime_error("partial_me: Incompatible dimensions");
    if (size % window_size == 0) return fold_axis_all(*this, u, size / window_size, window_size);
    // ragged last window: the reference treats missing elements as zero, so pad the flat tensor first
    const uint nwin = (size + window_size - 1) / window_size;
    FrTensor padded = FrTensor::filled(nwin * window_size, Fr_t{{0, 0, 0, 0, 0, 0, 0, 0}});
    ZKC(zk_memcpy_d2d(padded.gpu_data, gpu_data, sizeof(Fr_t) * (size_t)size, nullptr));
    return fold_axis_all(padded, u, nwin, window_size);
}

FrTensor FrTensor::partial_me(const vector<Fr_t>& u, uint cur_dim, uint window_size) const {
    if (cur_dim <= ((1u << u.size()) >> 1)) throw std::runtime_error("cur_dim <= ((1<<u.size()) >> 1)");
    if (cur_dim > (1u << u.size())) throw std::runtime_error("cur_dim > (1<<u.size())");
    return fold_axis_all(*this, u, cur_dim, window_size);
}

Fr_t FrTensor::multi_dim_me(const vector<vector<Fr_t>>& us, const vector<uint>& shape) const {
    if (shape.size() != us.size()) throw std::runtime_error("Incompatible dimensions");
    if (shape.size() == 0) return (*this)(0);
    if (shape.size() == 1) return (*this)(us[0]);
    FrTensor t_new = this->partial_me(us.back(), shape.back(), 1);
    return t_new.multi_dim_me({us.begin(), us.end() - 1}, {shape.begin(), shape.end() - 1});
}

std::pair<FrTensor, FrTensor> FrTensor::split(uint window_size) const {
    if (window_size < 1 || window_size >= size) throw std::runtime_error("Invalid window size.");
    // even windows -> first, odd windows -> second (fr-tensor.cu:562-585); done with two strided gathers
    uint num_window_in = (size + window_size - 1) / window_size;
    uint num_window_out = (num_window_in + 1) / 2;
    uint out_size = num_window_out * window_size;
    std::vector<uint32_t> idx0(out_size), idx1(out_size);
    FrTensor padded = FrTensor::filled(size + 1, Fr_t{{0, 0, 0, 0, 0, 0, 0, 0}});   // slot `size` reads as zero
    ZKC(zk_memcpy_d2d(padded.gpu_data, gpu_data, sizeof(Fr_t) * (size_t)size, nullptr));
    for (uint g = 0; g < out_size; ++g) {
        uint w = g / window_size, j = g % window_size;
        uint g0 = 2 * w * window_size + j, g1 = (2 * w + 1) * window_size + j;
        idx0[g] = g0 < size ? g0 : size;
        idx1[g] = g1 < size ? g1 : size;
    }
    DevBuf d0(sizeof(uint32_t) * (size_t)out_size), d1(sizeof(uint32_t) * (size_t)out_size);
    ZKC(zk_memcpy_h2d(d0.p, idx0.data(), sizeof(uint32_t) * (size_t)out_size, nullptr));
    ZKC(zk_memcpy_h2d(d1.p, idx1.data(), sizeof(uint32_t) * (size_t)out_size, nullptr));
    std::pair<FrTensor, FrTensor> out{FrTensor(out_size), FrTensor(out_size)};
    ZKC(zk_fr_gather(out.first.gpu_data, padded.gpu_data, d0.p, out_size, nullptr));
    ZKC(zk_fr_gather(out.second.gpu_data, padded.gpu_data, d1.p, out_size, nullptr));
    ZKC(zk_sync(nullptr));
    return out;
}

FrTensor FrTensor::pad(const vector<uint>& shape, const Fr_t& pad_val) const {
    size_t cum = 1;
    for (auto& s : shape) cum *= s;
    if (cum != size) throw std::runtime_error("pad: cum_shape != size");
    // fr-tensor.cu:800-828 pads the last dimension, merges it into the one before and repeats; a level whose length already
    // is a power of two changes nothing and takes no pass here
    vector<uint> sh(shape);
    std::unique_ptr<FrTensor> cur;
    for (;;) {
        const FrTensor& src = cur ? *cur : *this;
        const uint last_dim = sh.back(), last_dim_padded = 1u << ceilLog2(last_dim);
        if (last_dim != last_dim_padded) {
            const size_t rows = src.size / last_dim;
            std::unique_ptr<FrTensor> out(new FrTensor((uint)(rows * last_dim_padded)));
            ZKC(zk_fr_pad(out->gpu_data, src.gpu_data, rows, last_dim, last_dim_padded, pad_val.val, nullptr));
            cur = std::move(out);
        }
        if (sh.size() == 1) break;
        sh.pop_back();
        sh.back() *= last_dim_padded;
    }
    if (!cur) return FrTensor(*this);
    return FrTensor(std::move(*cur));
}

FrTensor FrTensor::transpose(uint M, uint N) const {
    if (size != M * N) throw std::runtime_error("transpose: incompatible dimensions");
    FrTensor out(N * M);
    ZKC(zk_fr_transpose(out.gpu_data, gpu_data, M, N, nullptr));
    return out;
}

FrTensor FrTensor::trunc(uint begin_idx, uint end_idx) const {
    if (begin_idx >= end_idx || end_idx > size) throw std::runtime_error("trunc: invalid indices");
    FrTensor out(end_idx - begin_idx);
    ZKC(zk_memcpy_d2d(out.gpu_data, gpu_data + begin_idx, sizeof(Fr_t) * (size_t)out.size, nullptr));
    return out;
}

FrTensor FrTensor::matmul(const FrTensor& x, const FrTensor& y, uint M, uint N, uint P) {
    if (x.size != M * N || y.size != N * P) throw std::runtime_error("matmul: incompatible dimensions");
    FrTensor out(M * P);
    int path = 0;
    MatmulRhsCache* rc = y.rhs_cache.get();
    if (rc && rc->prepared && (rc->N != N || rc->P != P)) rc->reset();       // the same elements read as another shape
    if (rc && !rc->prepared) {
        ZKC(zk_fr_matmul_rhs_prepare(&rc->prepared, y.gpu_data, N, P, nullptr));
        rc->N = N; rc->P = P;
    }
    // a left operand with an int32 form (a rescaled activation) is read from it, except where the caller asked for the generic product
    const void* xi = (rc && G().matmul_mode != 1) ? x.kept_ints() : nullptr;
    if (xi) ZKC(zk_fr_matmul_rhs_ints(out.gpu_data, zk_fr_fold_prepared_ints(xi), rc->prepared, M, G().matmul_mode, &path, nullptr));
    else if (rc) ZKC(zk_fr_matmul_rhs(out.gpu_data, x.gpu_data, rc->prepared, M, G().matmul_mode, &path, nullptr));
    else ZKC(zk_fr_matmul(out.gpu_data, x.gpu_data, y.gpu_data, M, N, P, G().matmul_mode, &path, nullptr));
    G().last_matmul_path = path;
    return out;
}

FrTensor FrTensor::transpose_stack(uint num, uint M, uint N) const {
    if ((size_t)size != (size_t)num * M * N) throw std::runtime_error("transpose: incompatible dimensions");
    FrTensor out(size);
    ZKC(zk_fr_transpose_batched(out.gpu_data, gpu_data, num, M, N, nullptr));
    return out;
}
FrTensor FrTensor::swap_leading_axes(uint A, uint B, uint C) const {
    if ((size_t)size != (size_t)A * B * C) throw std::runtime_error("swap_leading_axes: incompatible dimensions");
    FrTensor out(size);
    ZKC(zk_fr_swap_axes(out.gpu_data, gpu_data, A, B, C, nullptr));
    return out;
}
FrTensor FrTensor::matmul_stack(const FrTensor& x, const FrTensor& y, uint num, uint M, uint N, uint P) {
    FrTensor out(num * M * P);
    matmul_stack_into(out, x, y, num, M, N, P);
    return out;
}
FrTensor FrTensor::matmul_stack_prod(const FrTensor& a, const FrTensor& b, const FrTensor& y, uint num, uint M, uint N, uint P) {
    if ((size_t)a.size != (size_t)num * M * N || b.size != a.size || (size_t)y.size != (size_t)num * N * P) throw std::runtime_error("matmul: incompatible dimensions");
    if (!a.kept_ints() || !b.kept_ints()) throw std::runtime_error("matmul_stack_prod: both factors need an int32 form");
    FrTensor out(num * M * P);
    int path = 0;
    ZKC(zk_fr_matmul_batched_prod(out.gpu_data, zk_fr_fold_prepared_ints(a.kept_ints()), zk_fr_fold_prepared_ints(b.kept_ints()), y.gpu_data, num, M, N, P, G().matmul_mode, &path, nullptr));
    G().last_matmul_path = path;
    return out;
}
FrTensor FrTensor::partial_me_prod(const FrTensor& a, const FrTensor& b, const vector<Fr_t>& u, uint cur_dim, uint window_size) {
    if (a.size != b.size || !a.kept_ints() || !b.kept_ints()) throw std::runtime_error("partial_me_prod: two tensors of one size with int32 forms");
    if (u.empty() || u.size() > 24 || cur_dim <= ((1u << u.size()) >> 1) || cur_dim > (1u << u.size())) throw std::runtime_error("partial_me_prod: Incompatible dimensions");
    if ((size_t)a.size % ((size_t)cur_dim * window_size) != 0) throw std::runtime_error("t.size % (cur_dim * window_size) != 0");
    const size_t other = (size_t)a.size / ((size_t)cur_dim * window_size);
    FrTensor out((uint)(other * window_size));
    ZKC(zk_fr_fold_axis_prod(out.gpu_data, a.kept_ints(), b.kept_ints(), u[0].val, (int)u.size(), other, cur_dim, window_size, nullptr));
    return out;
}
void FrTensor::matmul_stack_into(FrTensor& out, const FrTensor& x, const FrTensor& y, uint num, uint M, uint N, uint P) {
    if ((size_t)x.size != (size_t)num * M * N || (size_t)y.size != (size_t)num * N * P || (size_t)out.size != (size_t)num * M * P)
        throw std::runtime_error("matmul: incompatible dimensions");
    int path = 0;
    ZKC(zk_fr_matmul_batched(out.gpu_data, x.gpu_data, y.gpu_data, num, M, N, P, G().matmul_mode, &path, nullptr));
    G().last_matmul_path = path;
}

// The reference draws these from cuRAND with a random_device seed (fr-tensor.cu:444-510); here they come
// from the seedable host stream: same distributions, reproducible.
FrTensor FrTensor::random_int(uint size, uint num_bits) {
    ensure_seeded();
    std::mt19937& mt = G().mt;
    std::vector<long> v(size);
    for (uint i = 0; i < size; ++i) v[i] = (long)((uint)mt() & ((1u << num_bits) - 1)) - (long)(1u << (num_bits - 1));
    return FrTensor(size, v.data());
}
FrTensor FrTensor::random(uint size) {
    vector<Fr_t> v = random_vec(size);
    return FrTensor(size, v.data());
}
FrTensor FrTensor::filled(uint size, const Fr_t& x) {
    FrTensor out(size);
    ZKC(zk_fr_fill(out.gpu_data, x.val, size, nullptr));
    return out;
}

ostream& operator<<(ostream& os, const FrTensor& A) {
    os << '[';
    for (uint i = 0; i + 1 < A.size; ++i) os << A(i) << '\n';
    os << A(A.size - 1) << ']';
    return os;
}

FrTensor catTensors(const vector<FrTensor>& vec) {
    uint size = vec[0].size;
    for (uint i = 1; i < vec.size(); i++)
        if (vec[i].size != size) throw std::runtime_error("tensor size does not match!");
    uint num = (uint)vec.size();
    FrTensor out(num * size);
    for (uint i = 0; i < num; i++)
        ZKC(zk_memcpy_d2d(out.gpu_data + (size_t)i * size, vec[i].gpu_data, (size_t)size * sizeof(Fr_t), nullptr));
    return out;
}

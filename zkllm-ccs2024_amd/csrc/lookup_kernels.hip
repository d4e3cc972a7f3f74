// Lookup argument, rescaling and softmax kernels for gfx950 (replaces the kernels of tlookup.cu,
// rescaling.cu, zksoftmax.cu and the multi-Hadamard kernels of proof.cu:172-188).
//
//  * multiplicities: indices are histogrammed into LDS-private counters when the table fits
//    (<= 16 Ki bins), otherwise with wave-aggregated global atomics, so a column of equal values
//    costs one atomic per wave instead of 64 (tlookup.cu:10-48 uses one global atomic per query).
//  * inverses: Montgomery's batch inversion across a whole 512-lane workgroup -- prefix and
//    suffix products through LDS and a single Fermat exponentiation per 4096 elements -- instead of
//    one 255-bit exponentiation per element (tlookup.cu:50-62).  Inverses are unique, so outputs
//    are identical; zero inputs give zero as 0^(r-2) does.
//  * sumcheck rounds: the multilinear evaluations of the per-round term tensors
//    (tlookup.cu:184-279) are taken as inner products with the eq(u, .) table, so one pass over
//    the operands yields every coefficient of the round polynomial and the folded operands; no
//    term tensor is ever written.
//  * softmax shift / exp tables use the deterministic exp/log of detmath.hpp.
#include <cstring>
#include <memory>
#include <vector>
#include "detmath.hpp"
#include "field.hpp"
#include "fr29.hpp"
#include <mutex>
#include <utility>
#include <vector>
#include "rt.hpp"
#include "../../include/zkllm_hip.h"

using namespace zk;

static constexpr int TPB = 256;
static inline Fr load_fr(const uint32_t* p) { Fr r; memcpy(&r, p, 32); return r; }
// Streamed operands of a kernel that also gathers from a table: loaded and stored past the caches' retention, so that the
// table's lines stay (elements are 32 bytes at 32-byte strides from 256-byte aligned blocks)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Fr ld_stream(const Fr* p) {
    const u32x4* q = (const u32x4*)p;
    const u32x4 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
    Fr r;
    r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w; r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
    return r;
}
__device__ __forceinline__ void st_stream(Fr* p, const Fr& x) {
    u32x4 a, b;
    a.x = x.v[0]; a.y = x.v[1]; a.z = x.v[2]; a.w = x.v[3]; b.x = x.v[4]; b.y = x.v[5]; b.z = x.v[6]; b.w = x.v[7];
    __builtin_nontemporal_store(a, (u32x4*)p);
    __builtin_nontemporal_store(b, (u32x4*)p + 1);
}

// ---- block reduction helper (K sums per thread) -------------------------------------------------------
template <int K> __device__ __forceinline__ void block_reduce_store(Fr (&acc)[K], Fr* __restrict__ partials) {
    __shared__ uint32_t red[8][TPB];
    const uint32_t t = threadIdx.x;
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int l = 0; l < 8; ++l) red[l][t] = acc[k].v[l];
        __syncthreads();
        for (uint32_t s = TPB / 2; s > 0; s >>= 1) {
            if (t < s) {
                Fr x, y;
#pragma unroll
                for (int l = 0; l < 8; ++l) { x.v[l] = red[l][t]; y.v[l] = red[l][t + s]; }
                x = add(x, y);
#pragma unroll
                for (int l = 0; l < 8; ++l) red[l][t] = x.v[l];
            }
            __syncthreads();
        }
        if (t == 0) {
            Fr x;
#pragma unroll
            for (int l = 0; l < 8; ++l) x.v[l] = red[l][0];
            partials[(size_t)k * gridDim.x + blockIdx.x] = x;
        }
        __syncthreads();
    }
}
__global__ void __launch_bounds__(TPB) k_finish(Fr* __restrict__ out, const Fr* __restrict__ partials, uint32_t nb) {
    Fr acc[1] = {big_zero<8>()};
    const Fr* p = partials + (size_t)blockIdx.x * nb;
    for (uint32_t i = threadIdx.x; i < nb; i += TPB) acc[0] = add(acc[0], p[i]);
    block_reduce_store<1>(acc, out);
}
// The partial sums of all rounds of a job at once, behind its last round: no round waits for the one before to be summed
// (the next round needs the fold challenge, not the sums).  Round r's K[r] sums: nb[r] partials each from part + off[r], into
// sums[r * per_round + k].  grid (most sums of a round, rounds)
static constexpr int FINISH_ROUNDS_MAX = 64;
struct FinishRounds { uint32_t off[FINISH_ROUNDS_MAX], nb[FINISH_ROUNDS_MAX]; uint8_t k[FINISH_ROUNDS_MAX]; };
struct PartSlice { Fr* p; template <class T> T* as() const { return reinterpret_cast<T*>(p); } };      // a round's share of the partial sums
__global__ void __launch_bounds__(TPB) k_finish_rounds(Fr* __restrict__ sums, const Fr* __restrict__ part, const FinishRounds fr, uint32_t per_round) {
    const uint32_t r = blockIdx.y;
    if (blockIdx.x >= fr.k[r]) return;
    Fr acc[1] = {big_zero<8>()};
    const uint32_t nb = fr.nb[r];
    const Fr* p = part + fr.off[r] + (size_t)blockIdx.x * nb;
    for (uint32_t i = threadIdx.x; i < nb; i += TPB) acc[0] = add(acc[0], p[i]);
    block_reduce_store<1>(acc, sums + (size_t)r * per_round);
}
static inline unsigned reduce_grid(size_t n) {
    size_t b = (n + TPB - 1) / TPB;
    if (b > 1024) b = 1024;
    if (b < 1) b = 1;
    return (unsigned)b;
}
// the grid of a round that gives a lane `per_lane` pairs where the round has them: at least 64 workgroups, at most reduce_grid's
static inline unsigned round_grid(size_t n, unsigned per_lane) {
    const size_t all = reduce_grid(n), want = n / ((size_t)TPB * per_lane);
    return (unsigned)std::min(all, std::max<size_t>(64, want));
}
// finish K sums (K x nb partials) and copy them to the host, applying the R correction (to_mont)
// to the first `n_mont` of them
static int finish_sums(Fr* partials, unsigned nb, int K, int n_mont, Fr* host_out, hipStream_t st) {
    void* stage = nullptr;
    int rc = staging(&stage, sizeof(Fr) * K);
    if (rc) return rc;
    Scratch fin(sizeof(Fr) * K, st);
    if (fin.rc) return fin.rc;
    hipLaunchKernelGGL(k_finish, dim3(K), dim3(TPB), 0, st, fin.as<Fr>(), partials, nb);
    ZK_LAUNCH_CHECK();
    (void)stage;
    return deliver(st, fin.p, host_out, (size_t)K, n_mont);
}

// ---- table index / histogram ---------------------------------------------------------------------------------
// idx = (val - low).val[0]  (lookuprange_tensor_prep_kernel tlookup.cu:414-421); an index outside the
// table (which the reference would use unchecked) raises the flag instead.
__global__ void __launch_bounds__(TPB) k_index_fr(uint32_t* __restrict__ idx, uint32_t* __restrict__ flag, const Fr* __restrict__ vals, const Fr low, uint32_t table_size, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const Fr d = sub(vals[i], low);
    const bool ok = !(d.v[1] | d.v[2] | d.v[3] | d.v[4] | d.v[5] | d.v[6] | d.v[7]) && d.v[0] < table_size;
    idx[i] = ok ? d.v[0] : 0u;
    if (!ok) atomicOr(flag, 1u);
}
__global__ void __launch_bounds__(TPB) k_index_i32(uint32_t* __restrict__ idx, uint32_t* __restrict__ flag, const int32_t* __restrict__ vals, int32_t low, uint32_t table_size, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int64_t d = (int64_t)vals[i] - (int64_t)low;
    const bool ok = d >= 0 && d < (int64_t)table_size;
    idx[i] = ok ? (uint32_t)d : 0u;
    if (!ok) atomicOr(flag, 1u);
}
// Where a counting pass takes its table positions from: an array of them, or the queries themselves in int32 form (position =
// value - low; a value outside [low, low + len) counts as position 0 and raises *flag in the passes that are asked to check).
struct KeySrc { const uint32_t* idx; const int32_t* vals; int32_t low; uint32_t len; uint32_t* flag; };
template <bool CHECK> __device__ __forceinline__ uint32_t key_at(const KeySrc& k, size_t i) {
    if (k.idx) return k.idx[i];
    const int64_t d = (int64_t)k.vals[i] - (int64_t)k.low;
    const bool ok = d >= 0 && d < (int64_t)k.len;
    if (CHECK && !ok) atomicOr(k.flag, 1u);
    return ok ? (uint32_t)d : 0u;
}
static constexpr uint32_t HIST_LDS_BINS = 16384;
__global__ void __launch_bounds__(TPB) k_hist_lds(uint32_t* __restrict__ counts, const KeySrc idx, size_t n, uint32_t nbins) {
    __shared__ uint32_t h[HIST_LDS_BINS];
    for (uint32_t b = threadIdx.x; b < nbins; b += TPB) h[b] = 0;
    __syncthreads();
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (size_t)gridDim.x * TPB) atomicAdd(&h[key_at<true>(idx, i)], 1u);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < nbins; b += TPB) {
        const uint32_t c = h[b];
        if (c) atomicAdd(&counts[b], c);
    }
}
// Large tables: a workgroup first counts its 4096 indices in a small hash table in LDS (key = bin, up to four probes)
// and touches global memory once per distinct bin it has seen; an index that finds its four slots taken by other
// bins goes to global memory directly.  Skewed inputs (digits of a narrow distribution: most indices in a few dozen
// bins) then cost a few dozen global atomics per workgroup instead of thousands on the same addresses; spread-out
// inputs fill the table and pay one global atomic per index, as they must.
static constexpr uint32_t HH_SLOTS = 1024, HH_PER_LANE = 16, HH_EMPTY = 0xFFFFFFFFu;
__global__ void __launch_bounds__(TPB) k_hist_global(uint32_t* __restrict__ counts, const KeySrc idx, size_t n) {
    __shared__ uint32_t keys[HH_SLOTS], cnts[HH_SLOTS];
    for (uint32_t s = threadIdx.x; s < HH_SLOTS; s += TPB) { keys[s] = HH_EMPTY; cnts[s] = 0; }
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * TPB * HH_PER_LANE;
#pragma unroll 4
    for (uint32_t k = 0; k < HH_PER_LANE; ++k) {
        const size_t i = base + (size_t)k * TPB + threadIdx.x;
        if (i >= n) break;
        const uint32_t key = key_at<true>(idx, i);
        const uint32_t h = (key * 2654435761u) >> 22;          // 10 bits
        bool placed = false;
#pragma unroll
        for (uint32_t p = 0; p < 4 && !placed; ++p) {
            const uint32_t slot = (h + p) & (HH_SLOTS - 1);
            const uint32_t prev = atomicCAS(&keys[slot], HH_EMPTY, key);
            if (prev == HH_EMPTY || prev == key) { atomicAdd(&cnts[slot], 1u); placed = true; }
        }
        if (!placed) atomicAdd(&counts[key], 1u);
    }
    __syncthreads();
    for (uint32_t s = threadIdx.x; s < HH_SLOTS; s += TPB) {
        const uint32_t key = keys[s];
        if (key != HH_EMPTY) atomicAdd(&counts[key], cnts[s]);
    }
}
// Large tables and many queries: global atomics are the cost of k_hist_global when the queries spread over the table
// (13 G/s).  Here the queries are first partitioned by their high bits -- per-tile sizes, one exclusive scan, a scatter of
// the low 12 bits as u16 -- and every partition is then counted in LDS, 4096 bins at a time, by as many workgroups as its
// size asks for; global memory sees one atomic per non-empty bin and slice.  Skewed inputs (one partition holding nearly
// everything) only make that partition's slices hit the same LDS counters, which an LDS serves far faster than L2 does.
static constexpr uint32_t HP_BITS = 12, HP_BINS = 1u << HP_BITS;   // bins per partition
static constexpr uint32_t HP_TILE = 65536;                           // queries per workgroup of the partition passes
static constexpr uint32_t HP_SLICE = 32768;                          // queries per workgroup of the counting pass
static constexpr uint32_t HP_MAXP = 1024;                            // partitions: tables up to 2^22 bins
static constexpr size_t HP_MIN_QUERIES = (size_t)1 << 20;
__global__ void __launch_bounds__(TPB) k_hp_sizes(uint32_t* __restrict__ sizes, const KeySrc idx, size_t n, uint32_t P, uint32_t ntiles) {
    __shared__ uint32_t c[HP_MAXP];
    for (uint32_t q = threadIdx.x; q < P; q += TPB) c[q] = 0;
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * HP_TILE, end = base + HP_TILE < n ? base + HP_TILE : n;
    for (size_t i = base + threadIdx.x; i < end; i += TPB) atomicAdd(&c[key_at<true>(idx, i) >> HP_BITS], 1u);
    __syncthreads();
    for (uint32_t q = threadIdx.x; q < P; q += TPB) sizes[(size_t)q * ntiles + blockIdx.x] = c[q];
}
// workgroup q: row q of the sizes (one entry per tile) -> its exclusive prefix sums; totals[q] = the row's sum
__global__ void __launch_bounds__(TPB) k_hp_rowscan(uint32_t* __restrict__ a, uint32_t* __restrict__ totals, uint32_t ntiles) {
    __shared__ uint32_t part[TPB];
    uint32_t* row = a + (size_t)blockIdx.x * ntiles;
    const uint32_t t = threadIdx.x;
    uint32_t carry = 0;
    for (uint32_t base = 0; base < ntiles; base += TPB) {
        const uint32_t i = base + t, v = i < ntiles ? row[i] : 0u;
        part[t] = v;
        __syncthreads();
        for (uint32_t off = 1; off < (uint32_t)TPB; off <<= 1) {
            const uint32_t x = t >= off ? part[t - off] : 0u;
            __syncthreads();
            part[t] += x;
            __syncthreads();
        }
        if (i < ntiles) row[i] = carry + part[t] - v;
        carry += part[TPB - 1];
        __syncthreads();
    }
    if (t == 0) totals[blockIdx.x] = carry;
}
// one workgroup: part_off[q] = where partition q starts (part_off[P] = n), and the list of (partition, slice) pairs the
// counting pass works through, slice_tab[k] = partition << 22 | slice
__global__ void __launch_bounds__(1024) k_hp_slices(uint32_t* __restrict__ slice_tab, uint32_t* __restrict__ nslices, uint32_t* __restrict__ part_off,
                                                    const uint32_t* __restrict__ totals, uint32_t P) {
    __shared__ uint32_t part[1024];
    const uint32_t t = threadIdx.x;
    const uint32_t size = t < P ? totals[t] : 0u;
    part[t] = size;
    __syncthreads();
    for (uint32_t off = 1; off < 1024u; off <<= 1) {
        const uint32_t v = t >= off ? part[t - off] : 0u;
        __syncthreads();
        part[t] += v;
        __syncthreads();
    }
    if (t < P) part_off[t] = part[t] - size;
    if (t == 1023u) part_off[P] = part[1023];
    __syncthreads();
    const uint32_t ns = (size + HP_SLICE - 1) / HP_SLICE;
    part[t] = ns;
    __syncthreads();
    for (uint32_t off = 1; off < 1024u; off <<= 1) {
        const uint32_t v = t >= off ? part[t - off] : 0u;
        __syncthreads();
        part[t] += v;
        __syncthreads();
    }
    const uint32_t o = part[t] - ns;
    for (uint32_t q = 0; q < ns; ++q) slice_tab[o + q] = (t << 22) | q;
    if (t == 1023u) *nslices = part[1023];
}
__global__ void __launch_bounds__(TPB) k_hp_scatter(uint16_t* __restrict__ parted, const uint32_t* __restrict__ offs, const uint32_t* __restrict__ part_off,
                                                    const KeySrc idx, size_t n, uint32_t P, uint32_t ntiles) {
    __shared__ uint32_t cur[HP_MAXP];
    for (uint32_t q = threadIdx.x; q < P; q += TPB) cur[q] = part_off[q] + offs[(size_t)q * ntiles + blockIdx.x];
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * HP_TILE, end = base + HP_TILE < n ? base + HP_TILE : n;
    for (size_t i = base + threadIdx.x; i < end; i += TPB) {
        const uint32_t key = key_at<false>(idx, i);
        const uint32_t pos = atomicAdd(&cur[key >> HP_BITS], 1u);
        parted[pos] = (uint16_t)(key & (HP_BINS - 1u));
    }
}
__global__ void __launch_bounds__(TPB) k_hp_count(uint32_t* __restrict__ counts, const uint16_t* __restrict__ parted, const uint32_t* __restrict__ part_off,
                                                  const uint32_t* __restrict__ slice_tab, const uint32_t* __restrict__ nslices, uint32_t nbins) {
    if (blockIdx.x >= *nslices) return;
    __shared__ uint32_t h[HP_BINS];
    const uint32_t e = slice_tab[blockIdx.x], q = e >> 22, sl = e & ((1u << 22) - 1u);
    for (uint32_t b = threadIdx.x; b < HP_BINS; b += TPB) h[b] = 0;
    __syncthreads();
    const uint32_t start = part_off[q] + sl * HP_SLICE, stop = part_off[q + 1];
    const uint32_t end = stop - start > HP_SLICE ? start + HP_SLICE : stop;
    for (uint32_t i = start + threadIdx.x; i < end; i += TPB) atomicAdd(&h[parted[i]], 1u);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < HP_BINS; b += TPB) {
        const uint32_t c = h[b], bin = q * HP_BINS + b;
        if (c && bin < nbins) atomicAdd(&counts[bin], c);
    }
}
static int hist_partitioned(uint32_t* counts, const KeySrc idx, size_t n, uint32_t nbins, hipStream_t st) {
    const uint32_t P = (nbins + HP_BINS - 1) / HP_BINS, ntiles = cdiv(n, HP_TILE), M = P * ntiles;
    const uint32_t max_slices = (uint32_t)(n / HP_SLICE) + P + 1;
    Scratch sizes(sizeof(uint32_t) * (size_t)M, st), part_off(sizeof(uint32_t) * (P + 1), st), totals(sizeof(uint32_t) * P, st), slice_tab(sizeof(uint32_t) * max_slices, st),
        nsl(sizeof(uint32_t), st), parted(sizeof(uint16_t) * n, st);
    for (const Scratch* b : {&sizes, &part_off, &totals, &slice_tab, &nsl, &parted})
        if (b->rc) return b->rc;
    hipLaunchKernelGGL(k_hp_sizes, dim3(ntiles), dim3(TPB), 0, st, sizes.as<uint32_t>(), idx, n, P, ntiles);
    hipLaunchKernelGGL(k_hp_rowscan, dim3(P), dim3(TPB), 0, st, sizes.as<uint32_t>(), totals.as<uint32_t>(), ntiles);
    hipLaunchKernelGGL(k_hp_slices, dim3(1), dim3(1024), 0, st, slice_tab.as<uint32_t>(), nsl.as<uint32_t>(), part_off.as<uint32_t>(), totals.as<uint32_t>(), P);
    hipLaunchKernelGGL(k_hp_scatter, dim3(ntiles), dim3(TPB), 0, st, parted.as<uint16_t>(), sizes.as<uint32_t>(), part_off.as<uint32_t>(), idx, n, P, ntiles);
    hipLaunchKernelGGL(k_hp_count, dim3(max_slices), dim3(TPB), 0, st, counts, parted.as<uint16_t>(), part_off.as<uint32_t>(), slice_tab.as<uint32_t>(), nsl.as<uint32_t>(), nbins);
    ZK_LAUNCH_CHECK();
    return 0;
}
// table[i] = low + min(i, len-1)  (tlookuprange_init_kernel tlookup.cu:372-380)
__global__ void __launch_bounds__(TPB) k_range_table(Fr* __restrict__ table, int32_t low, uint32_t len, uint32_t table_size) {
    const uint32_t t = blockIdx.x * TPB + threadIdx.x;
    if (t >= table_size) return;
    const int64_t v = (t < len) ? (int64_t)t + low : (int64_t)len + low - 1;
    table[t] = fr_from_i64(v);
}

// ---- batch inversion -----------------------------------------------------------------------------------------------
// out[i] = 1 / (in[i] + beta), 0 where the sum is 0.  A workgroup inverts T * 8 values with one field inversion:
// every lane multiplies its 8 values up, the T lane products go up a product tree in LDS, the root is inverted, and
// the inverse comes down the tree (a child's inverse is the parent's inverse times the sibling) and through each
// lane's values backwards.  About 3.4 multiplications per value.
// The standard-form inputs are used as they are: x is the Montgomery representation of x/R, every product of the
// scheme is then a Montgomery representation too, and the two stray factors of R in each result are removed once per
// workgroup by multiplying the root's inverse by R^-1 (a Montgomery product with R^-1 multiplies by R^-2).
//
// One field inversion is a serial computation of about 140 us on one lane, during which the rest of its workgroup
// waits with its registers held.  Large inputs therefore run in three steps (MODE): BI_UP only multiplies up to the
// workgroup's root and writes it to roots[workgroup]; the roots -- a few thousand numbers -- are inverted by this same
// scheme (the corrected inverse of a root is exactly the plain inverse of the number written); BI_DOWN repeats the
// way up, takes its root's inverse from roots_inv[workgroup] and comes down.  The two large steps then have no serial part.
enum { BI_FULL = 0, BI_UP = 1, BI_DOWN = 2 };
static constexpr int BI_T = 512, BI_CH = 8;        // single-step form (small inputs)
static constexpr int BI_T3 = 256;                  // three-step form
template <int T, int MODE>
__global__ void __launch_bounds__(T) k_batch_inv(Fr* __restrict__ out, const Fr* __restrict__ in, const Fr beta, size_t n, Fr* __restrict__ roots, const Fr* __restrict__ roots_inv) {
    __shared__ uint32_t node[8][2 * T];      // level 0 (lane products) at [0, T), level 1 at [T, T + T/2), ... root at 2T - 2
    const uint32_t t = threadIdx.x;
    const size_t base = ((size_t)blockIdx.x * T + t) * BI_CH;
    const Fr one_m = big_one_mont<8>();
    Fr x[BI_CH], pre[BI_CH];
    uint32_t nz = 0;
    Fr tot = one_m;
#pragma unroll
    for (int c = 0; c < BI_CH; ++c) {
        Fr v = big_zero<8>();
        if (base + c < n) v = add(in[base + c], beta);
        const bool nzc = !is_zero(v);
        nz |= (nzc ? 1u : 0u) << c;
        x[c] = nzc ? v : one_m;
        pre[c] = tot;
        tot = mont_mul(tot, x[c]);
    }
    auto put = [&](const Fr& v, uint32_t i) {
#pragma unroll
        for (int l = 0; l < 8; ++l) node[l][i] = v.v[l];
    };
    auto get = [&](uint32_t i) {
        Fr v;
#pragma unroll
        for (int l = 0; l < 8; ++l) v.v[l] = node[l][i];
        return v;
    };
    put(tot, t);
    __syncthreads();
    // up: level L has T >> L nodes starting at off(L) = 2*T - (2*T >> L)
    uint32_t off = 0;
    for (uint32_t cnt = T / 2; cnt >= 1; cnt >>= 1) {
        const uint32_t noff = off + 2 * cnt;
        if (t < cnt) put(mont_mul(get(off + 2 * t), get(off + 2 * t + 1)), noff + t);
        __syncthreads();
        off = noff;
    }
    // off is now the root's index
    if (MODE == BI_UP) {
        if (t == 0) roots[blockIdx.x] = get(off);
        return;
    }
    if (MODE == BI_DOWN) {
        if (t == 0) put(roots_inv[blockIdx.x], off);
    } else if (t < 64) {
        Fr inv = mont_inverse(get(off));
        constexpr uint32_t RINV[8] = {4269129792u, 334977897u, 165441631u, 2876230287u, 1333208682u, 1912866698u, 805346647u, 465471123u};   // R^-1 mod r
        Fr k;
#pragma unroll
        for (int l = 0; l < 8; ++l) k.v[l] = RINV[l];
        inv = mont_mul(inv, k);
        if (t == 0) put(inv, off);
    }
    __syncthreads();
    // down: the inverse of a node replaces its value; a child reads the parent's inverse and its sibling's value first
    for (uint32_t cnt = 1; cnt < (uint32_t)T; cnt <<= 1) {
        const uint32_t coff = off - 2 * cnt;          // children level: 2*cnt nodes
        Fr inv_c = one_m;
        if (t < 2 * cnt) inv_c = mont_mul(get(off + (t >> 1)), get(coff + (t ^ 1u)));
        __syncthreads();
        if (t < 2 * cnt) put(inv_c, coff + t);
        __syncthreads();
        off = coff;
    }
    Fr inv_run = get(t);
#pragma unroll
    for (int c = BI_CH - 1; c >= 0; --c) {
        const Fr inv_c = mont_mul(inv_run, pre[c]);
        inv_run = mont_mul(inv_run, x[c]);
        if (base + c < n) out[base + c] = ((nz >> c) & 1u) ? inv_c : big_zero<8>();
    }
}
// queues out = 1 / (in + beta) on st; scratch comes from the arena, which must outlive the launches
static int batch_inv_queue(Fr* out, const Fr* in, const Fr& beta, size_t n, Arena& arena, hipStream_t st) {
    if (n == 0) return 0;
    if (n <= (size_t)2 * BI_T * BI_CH) {
        hipLaunchKernelGGL((k_batch_inv<BI_T, BI_FULL>), dim3(cdiv(n, (size_t)BI_T * BI_CH)), dim3(BI_T), 0, st, out, in, beta, n, (Fr*)nullptr, (const Fr*)nullptr);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    const size_t m = cdiv(n, (size_t)BI_T3 * BI_CH);
    Scratch& roots = arena.add(sizeof(Fr) * 2 * m);
    if (roots.rc) return roots.rc;
    Fr* r = roots.as<Fr>();
    hipLaunchKernelGGL((k_batch_inv<BI_T3, BI_UP>), dim3(m), dim3(BI_T3), 0, st, (Fr*)nullptr, in, beta, n, r, (const Fr*)nullptr);
    ZK_LAUNCH_CHECK();
    int rc = batch_inv_queue(r + m, r, big_zero<8>(), m, arena, st);
    if (rc) return rc;
    hipLaunchKernelGGL((k_batch_inv<BI_T3, BI_DOWN>), dim3(m), dim3(BI_T3), 0, st, out, in, beta, n, (Fr*)nullptr, (const Fr*)(r + m));
    ZK_LAUNCH_CHECK();
    return 0;
}

// ---- eq tables ----------------------------------------------------------------------------------------------------------
// E[t] = prod_j (u_j if bit_j(t) else 1-u_j), Montgomery form.  Built by doubling: level j appends bit j.
__global__ void __launch_bounds__(TPB) k_eq_double(Fr* __restrict__ e, const Fr u_mont, const Fr one_minus_u_mont, size_t half) {
    const size_t t = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (t >= half) return;
    const Fr x = e[t];
    e[t + half] = mont_mul(x, u_mont);
    e[t] = mont_mul(x, one_minus_u_mont);
}
// dropping the top variable: E'[t] = E[t] + E[t + n_out]
__global__ void __launch_bounds__(TPB) k_eq_halve(Fr* __restrict__ out, const Fr* __restrict__ in, size_t n_out) {
    const size_t t = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (t < n_out) out[t] = add(in[t], in[t + n_out]);
}

// The table in two launches instead of one per variable: small tables over the low and the high half of the variables
// (every entry is a product of at most 15 factors), then their outer product.
struct EqChallenges { Fr u[30], omu[30]; };     // u_j and 1 - u_j, Montgomery form
__global__ void __launch_bounds__(TPB) k_eq_halves(Fr* __restrict__ lo, Fr* __restrict__ hi, const EqChallenges c, int kl, int kh) {
    const uint32_t g = blockIdx.x * TPB + threadIdx.x;
    const uint32_t nlo = 1u << kl, nhi = 1u << kh;
    if (g >= nlo + nhi) return;
    const bool is_hi = g >= nlo;
    const uint32_t t = is_hi ? g - nlo : g;
    const int first = is_hi ? kl : 0, cnt = is_hi ? kh : kl;
    Fr e = big_one_mont<8>();
    for (int j = 0; j < cnt; ++j) e = mont_mul(e, ((t >> j) & 1u) ? c.u[first + j] : c.omu[first + j]);
    (is_hi ? hi : lo)[t] = e;
}
__global__ void __launch_bounds__(TPB) k_eq_outer(Fr* __restrict__ e, const Fr* __restrict__ lo, const Fr* __restrict__ hi, int kl, size_t n) {
    const size_t t = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (t < n) e[t] = mont_mul(lo[t & ((1u << kl) - 1u)], hi[t >> kl]);
}

// Multilinear evaluations of up to 8 tensors at one point: a single pass that reads the point's eq table once and
// every tensor once (Fr_me, fr-tensor.cu:602-609, run once per tensor in the reference).  E carries R, each product
// one R^-1: the sums come out in standard form.
struct MePtrs { const Fr* x[8]; };
template <int K> __global__ void __launch_bounds__(TPB) k_me_multi(Fr* __restrict__ partials, const MePtrs p, const Fr* __restrict__ E, size_t n) {
    Fr acc[K];
#pragma unroll
    for (int k = 0; k < K; ++k) acc[k] = big_zero<8>();
    // four positions per step: their products with the eq entries share one Montgomery reduction (mont_dot)
    const size_t stride = (size_t)gridDim.x * TPB;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n; t += 4 * stride) {
        Fr e[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) e[j] = (t + j * stride < n) ? E[t + j * stride] : big_zero<8>();
#pragma unroll
        for (int k = 0; k < K; ++k) {
            Fr x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = (t + j * stride < n) ? p.x[k][t + j * stride] : big_zero<8>();
            acc[k] = add(acc[k], mont_dot<8, 4>(e, x));
        }
    }
    block_reduce_store<K>(acc, partials);
}

// 1 / (S[i] + beta) when every S[i] is expected to be a table entry: if S[i] equals T[j] for the hinted position
// j = hint[i] - low, the inverse is B[j] = 1 / (T[j] + beta), already computed for the table -- one gather instead of a
// share of a batch inversion over all D queries.  Whatever the hint, the result is the inverse itself: a query that
// does not match its hinted entry (a hint outside the table, inconsistent inputs) is inverted on its own.
// S_out != nullptr: the queries themselves are not stored; query i is hint[i] + r * S_out[i] (a mapping table's combined
// query, r_mont = r in Montgomery form) and is formed where it is needed.
// TB: table entry j and its inverse side by side, TB[2j] = T[j], TB[2j+1] = 1 / (T[j] + beta): the comparison and the
// inverse of one query come out of one 64-byte line (two gathers into separate arrays fetched two).
// hint_ints != nullptr (first round of a large job only): the queries are given by their int32 forms -- query i is
// hint_ints[i] (+ r * sout_ints[i] for a mapping table) and is never formed: where entry j = hint_ints[i] - low of the table
// is what these integers say (want[j], written by k_lookup_ints_check: the mapped integer of a consistent entry, 0 for a
// consistent entry of a plain table, INTS_POISON for an entry that is something else), query and inverse are TB[2j], TB[2j+1].
struct HintSrc { const Fr* TB; const Fr* hint; Fr low; Fr beta; uint32_t N; const Fr* S_out = nullptr; Fr r_mont;
                 const int32_t* hint_ints = nullptr; const int32_t* sout_ints = nullptr; const int32_t* want = nullptr; int32_t low_int = 0;
                 // *n_ok: the first table entry that is not what the integers say (k_lookup_ints_check; 0xFFFFFFFF: none) -- every entry
                 // below it is consistent, whatever lies above (a range table padded by repeating its last value is consistent up
                 // to its own length).  trusted_out: the outputs were gathered from this table by these queries
                 // (zk_fr_gather_by_queries_ints).  A query that names an entry below *n_ok then needs neither its output nor the
                 // entry's expected integer (for a plain table; for a mapping table with trusted outputs): nothing is gathered but
                 // the table record.
                 const uint32_t* n_ok = nullptr; bool trusted_out = false; };
static constexpr int32_t INTS_POISON = (int32_t)0x80000000;
__device__ __forceinline__ Fr hinted_query(const Fr* __restrict__ S, size_t i, const HintSrc& h) {
    return h.S_out ? add(h.hint[i], mont_mul(h.r_mont, h.S_out[i])) : S[i];
}
// Operands by value: a reference would have the caller keep every query in private memory ahead of the rarely taken call
// (64 bytes of private-memory stores per pair of the round kernel).
static __device__ __attribute__((noinline)) Fr inv_plus_beta_alone(const Fr sv, const Fr beta) {
    const Fr v = add(sv, beta);
    if (is_zero(v)) return big_zero<8>();
    // v is the Montgomery form of v/R: its Montgomery inverse is R^2/v, and a Montgomery product with R^-1 leaves 1/v
    constexpr uint32_t RINV[8] = {4269129792u, 334977897u, 165441631u, 2876230287u, 1333208682u, 1912866698u, 805346647u, 465471123u};
    Fr k;
#pragma unroll
    for (int l = 0; l < 8; ++l) k.v[l] = RINV[l];
    return mont_mul(mont_inverse(v), k);
}
// *unit (optional): the returned a satisfies a * (sv + beta) == 1 by construction (the hinted entry matched and is invertible)
__device__ __forceinline__ Fr inv_by_hint(const Fr& sv, size_t i, const HintSrc& h, bool* unit = nullptr) {
    const Fr d = sub(h.hint[i], h.low);
    const bool in_table = !(d.v[1] | d.v[2] | d.v[3] | d.v[4] | d.v[5] | d.v[6] | d.v[7]) && d.v[0] < h.N;
    const uint32_t j = in_table ? d.v[0] : 0u;
    if (equal(sv, h.TB[2 * (size_t)j])) {
        const Fr b = h.TB[2 * (size_t)j + 1];
        if (unit) *unit = !is_zero(b);
        return b;
    }
    if (unit) *unit = false;
    return inv_plus_beta_alone(sv, h.beta);
}
// want[j] for the int32 path of the first round: TB[2j] must be low + j (+ r * mapped[j])
__global__ void __launch_bounds__(TPB) k_lookup_ints_check(int32_t* __restrict__ want, uint32_t* __restrict__ n_ok, const Fr* __restrict__ TB,
                                                           const int32_t* __restrict__ mapped_ints, const Fr r_mont, int32_t low, uint32_t N) {
    const uint32_t j = blockIdx.x * TPB + threadIdx.x;
    if (j >= N) return;
    Fr q = fr_from_i64((int64_t)low + (int64_t)j);
    if (mapped_ints) q = add(q, mont_mul(r_mont, fr_from_i64((int64_t)mapped_ints[j])));
    const bool ok = equal(q, TB[2 * (size_t)j]) && (!mapped_ints || mapped_ints[j] != INTS_POISON);
    want[j] = ok ? (mapped_ints ? mapped_ints[j] : 0) : INTS_POISON;
    if (!ok) atomicMin(n_ok, j);          // *n_ok starts at 0xFFFFFFFF
}
// query i and 1 / (query + beta) from the int32 forms (HintSrc); unit as in inv_by_hint
__device__ __forceinline__ Fr query_inv_ints(size_t i, const HintSrc& h, Fr& a, bool& unit, int32_t* query = nullptr) {
    const int32_t hi = __builtin_nontemporal_load(h.hint_ints + i);
    if (query) *query = hi;
    const int64_t d = (int64_t)hi - (int64_t)h.low_int;
    const bool in_table = d >= 0 && d < (int64_t)h.N;
    const uint32_t j = in_table ? (uint32_t)d : 0u;
    const bool sure = in_table && j < *h.n_ok && (!h.sout_ints || h.trusted_out);
    int32_t so = 0;
    bool match = sure;
    if (!sure) {
        so = h.sout_ints ? __builtin_nontemporal_load(h.sout_ints + i) : 0;
        const int32_t w = h.want[j];
        match = in_table && w != INTS_POISON && so == w;
    }
    if (match) {
        a = h.TB[2 * (size_t)j + 1];
        unit = !is_zero(a);
        return h.TB[2 * (size_t)j];
    }
    Fr sv = fr_from_i64((int64_t)hi);
    if (h.sout_ints) sv = add(sv, mont_mul(h.r_mont, fr_from_i64((int64_t)so)));
    a = inv_plus_beta_alone(sv, h.beta);
    unit = false;
    return sv;
}
__global__ void __launch_bounds__(TPB) k_interleave(Fr* __restrict__ out, const Fr* __restrict__ a, const Fr* __restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) { out[2 * i] = a[i]; out[2 * i + 1] = b[i]; }
}
__global__ void __launch_bounds__(TPB) k_inv_by_hint(Fr* __restrict__ A, const Fr* __restrict__ S, const HintSrc h, size_t D) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < D) A[i] = inv_by_hint(S[i], i, h);
}
// out = a + r * b (the combined queries of a mapping table written out, for jobs too small for the fused first round)
__global__ void __launch_bounds__(TPB) k_combine_queries(Fr* __restrict__ out, const Fr* __restrict__ a, const Fr* __restrict__ b, const Fr r_mont, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = add(a[i], mont_mul(r_mont, b[i]));
}

// ---- lookup sumcheck round --------------------------------------------------------------------------------------------------
// Over halves (t, t + n_out):  a0 = A[t], da = A[t+n_out]-A[t], s0 = S[t]+beta, ds = S[t+n_out]-S[t]
//   sums 0..2 : sum E[t] * {a0 s0, da s0 + a0 ds, da ds}          (R^-1 attached)
//   sums 3..4 : sum a0, sum da
// phase 2 adds the same three E-weighted sums for (B,T) as sums 5..7 and the plain products of (m,B)
// as sums 8..10 (R^-1 attached), and folds all five tensors by v.
// HINTED (first round of a job whose A was never written): a0, a1 come from inv_by_hint instead of A.  Where both are
// inverses by construction (a0 s0 = a1 s1' = 1, s1' = S[t+n_out]+beta), the three E-weighted terms are 1, M - 4 and 4 - M
// with M = (a0 + a1)(s0 + s1'): one product instead of five, and the constants go through the sum of E.
template <bool PHASE2, bool HINTED = false> __global__ void __launch_bounds__(TPB)
k_lookup_round(Fr* __restrict__ partials, Fr* __restrict__ nA, Fr* __restrict__ nS, Fr* __restrict__ nB, Fr* __restrict__ nT, Fr* __restrict__ nm,
               const Fr* __restrict__ A, const Fr* __restrict__ S, const Fr* __restrict__ B, const Fr* __restrict__ T, const Fr* __restrict__ m,
               const Fr* __restrict__ E, const Fr beta, const Fr v_mont, size_t n_out, Fr* __restrict__ nE, const HintSrc hs = HintSrc()) {
    constexpr int K = PHASE2 ? 11 : 5;
    constexpr bool WIDE = !PHASE2;      // phase 1: the E-weighted products are summed unreduced, one reduction per lane (wide_redc)
    Fr acc[K];
#pragma unroll
    for (int i = 0; i < K; ++i) acc[i] = big_zero<8>();
    Fr acc_e = big_zero<8>(), acc_em = big_zero<8>();       // HINTED: sum of E and of E * M over the pairs of unit inverses
    WideAcc w0 = wide_zero(), w2 = wide_zero(), wx = wide_zero();      // sums of c0, c2 and of the cross products (a0 + da)(s0 + ds) E; HINTED: wx alone, the sum of E * M
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        const Fr e = HINTED ? ld_stream(E + t) : E[t];
        if (nE && t < n_out / 2) {      // the next round's table: the top variable summed out
            if (HINTED) st_stream(nE + t, add(e, ld_stream(E + t + n_out / 2)));
            else nE[t] = add(e, E[t + n_out / 2]);
        }
        {
            Fr s0r, s1, a0, a1;
            bool unit0 = false, unit1 = false;
            if (HINTED && hs.hint_ints) {
                s0r = query_inv_ints(t, hs, a0, unit0);
                s1 = query_inv_ints(t + n_out, hs, a1, unit1);
            } else {
                s0r = HINTED ? hinted_query(S, t, hs) : S[t];
                s1 = HINTED ? hinted_query(S, t + n_out, hs) : S[t + n_out];
                a0 = HINTED ? inv_by_hint(s0r, t, hs, &unit0) : A[t];
                a1 = HINTED ? inv_by_hint(s1, t + n_out, hs, &unit1) : A[t + n_out];
            }
            const Fr da = sub(a1, a0), ds = sub(s1, s0r), s0 = add(s0r, beta);
            if (HINTED && unit0 && unit1) {
                const Fr M = mont_mul(add(a0, a1), add(s0, add(s1, beta)));
                if constexpr (WIDE) wide_mac(wx, e, M);
                else acc_em = add(acc_em, mont_mul(e, M));
                acc_e = add(acc_e, e);
            } else {
                // E goes onto a0 and da first, and the middle term comes from (a0 + da)(s0 + ds): five products for the
                // three weighted terms instead of seven
                const Fr ea0 = mont_mul(e, a0), eda = mont_mul(e, da);
                if constexpr (WIDE && !HINTED) {
                    wide_mac(w0, ea0, s0);
                    wide_mac(w2, eda, ds);
                    wide_mac(wx, add(ea0, eda), add(s0, ds));
                } else {
                    // (HINTED: rare, a pair whose inverses did not both come from the table)
                    const Fr c0 = mont_mul(ea0, s0), c2 = mont_mul(eda, ds);
                    acc[0] = add(acc[0], c0);
                    acc[1] = add(acc[1], sub(sub(mont_mul(add(ea0, eda), add(s0, ds)), c0), c2));
                    acc[2] = add(acc[2], c2);
                }
            }
            acc[3] = add(acc[3], a0);
            acc[4] = add(acc[4], da);
            if (HINTED) {
                st_stream(nA + t, add(a0, mont_mul(v_mont, da)));
                st_stream(nS + t, add(s0r, mont_mul(v_mont, ds)));
            } else {
                nA[t] = add(a0, mont_mul(v_mont, da));
                nS[t] = add(s0r, mont_mul(v_mont, ds));
            }
        }
        if (PHASE2) {
            const Fr b0 = B[t], b1 = B[t + n_out], t0r = T[t], t1 = T[t + n_out], m0 = m[t], m1 = m[t + n_out];
            const Fr db = sub(b1, b0), dt = sub(t1, t0r), t0 = add(t0r, beta), dm = sub(m1, m0);
            const Fr eb0 = mont_mul(e, b0), edb = mont_mul(e, db);
            const Fr c5 = mont_mul(eb0, t0), c7 = mont_mul(edb, dt);
            acc[5] = add(acc[5], c5);
            acc[6] = add(acc[6], sub(sub(mont_mul(add(eb0, edb), add(t0, dt)), c5), c7));
            acc[7] = add(acc[7], c7);
            const Fr k0 = mont_mul(m0, b0), k2 = mont_mul(dm, db);
            acc[8] = add(acc[8], k0);
            acc[9] = add(acc[9], sub(sub(mont_mul(m1, b1), k0), k2));          // dm b0 + m0 db = m1 b1 - m0 b0 - dm db
            acc[10] = add(acc[10], k2);
            nB[t] = add(b0, mont_mul(v_mont, db));
            nT[t] = add(t0r, mont_mul(v_mont, dt));
            nm[t] = add(m0, mont_mul(v_mont, dm));
        }
    }
    if constexpr (WIDE && HINTED) acc_em = wide_redc(wx);
    if constexpr (WIDE && !HINTED) {
        acc[0] = wide_redc(w0);
        acc[2] = wide_redc(w2);
        acc[1] = sub(sub(wide_redc(wx), acc[0]), acc[2]);
    }
    if (HINTED) {
        // E is in Montgomery form and the sums carry R^-1: sum(E) * R^-2 through one product with R^-1
        constexpr uint32_t RINV[8] = {4269129792u, 334977897u, 165441631u, 2876230287u, 1333208682u, 1912866698u, 805346647u, 465471123u};
        Fr k;
#pragma unroll
        for (int l = 0; l < 8; ++l) k.v[l] = RINV[l];
        const Fr one = mont_mul(acc_e, k), two = add(one, one), four = add(two, two);
        acc[0] = add(acc[0], one);
        acc[1] = add(acc[1], sub(acc_em, four));
        acc[2] = add(acc[2], sub(four, acc_em));
    }
    block_reduce_store<K>(acc, partials);
}

// ---- the same round with the arithmetic in 29-bit limbs (fr29.hpp) ----------------------------------------------------------
// sum of up to 2^32 - 1 canonical elements as a plain 288-bit integer (nine words), and its residue
__device__ __forceinline__ void sum9_add(uint32_t (&acc)[9], const Fr& x) {
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = addc32(acc[i], x.v[i], c);
    acc[8] += c;
}
__device__ __forceinline__ Fr sum9_residue(const uint32_t (&acc)[9]) {
    Fr lo, hi = big_zero<8>();
#pragma unroll
    for (int i = 0; i < 8; ++i) lo.v[i] = acc[i];
    lo = reduce_once(reduce_once(lo));          // below 2^256 < 3 r
    hi.v[0] = acc[8];
    return add(lo, mont_mul(hi, big_r2<8>()));  // hi * 2^256
}
// k_lookup_round<false, false> (phase 1, inverses given) for rounds of many pairs: same inputs, same outputs (folded tensors
// canonical, the five sums as that kernel leaves them), about a quarter fewer vector instructions.  The eq weight e arrives
// as E 2^256: e a0 and e da come out as E a0 / 32 and E da / 32, the three sums of products are kept unreduced (Wide29),
// reduced once per lane (another 2^-261) and brought to the factor 2^-256 of the other kernel by one product with 2^271.
// At most 256 pairs per lane (the unreduced sums hold 2^522): the launch site checks.
__global__ void __launch_bounds__(TPB) k_lookup_round29(Fr* __restrict__ partials, Fr* __restrict__ nA, Fr* __restrict__ nS, const Fr* __restrict__ A, const Fr* __restrict__ S,
                                                        const Fr* __restrict__ E, const Fr beta, const Fr v_mont, size_t n_out, Fr* __restrict__ nE) {
    const Fr29 vq = fr29_mul(fr29_repack(v_mont), fr29_2_266());      // v 2^261
    const Fr29 b29 = fr29_repack(beta);
    Wide29 w0 = wide29_zero(), w2 = wide29_zero(), wx = wide29_zero();
    uint32_t sa0[9], sa1[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) sa0[i] = sa1[i] = 0;
    uint32_t it = 0;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        const Fr e = E[t];
        if (nE && t < n_out / 2) nE[t] = add(e, E[t + n_out / 2]);      // the next round's table: the top variable summed out
        const Fr a0w = A[t], a1w = A[t + n_out], s0w = S[t], s1w = S[t + n_out];
        sum9_add(sa0, a0w);
        sum9_add(sa1, a1w);
        const Fr29 e29 = fr29_repack(e), a0 = fr29_repack(a0w), s0r = fr29_repack(s0w);
        const Fr29 da = fr29_sub_plus_r(fr29_repack(a1w), a0), ds = fr29_sub_plus_r(fr29_repack(s1w), s0r);      // + r: non-negative, the same residues
        const Fr29 s0 = fr29_add(s0r, b29);
        const Fr29 ea0 = fr29_mul(e29, a0), eda = fr29_mul(e29, da);
        wide29_mac(w0, ea0, s0);
        wide29_mac(w2, eda, ds);
        wide29_mac(wx, fr29_add(ea0, eda), fr29_add(s0, ds));
        if ((++it & 3u) == 0u) { wide29_carry(w0); wide29_carry(w2); wide29_carry(wx); }
        nA[t] = fr29_canon_pack(fr29_add(a0, fr29_mul(vq, da)));
        nS[t] = fr29_canon_pack(fr29_add(s0r, fr29_mul(vq, ds)));
    }
    Fr acc[5];
    const Fr29 fix = fr29_2_271();
    acc[0] = fr29_canon_pack(fr29_mul(wide29_redc(w0), fix));
    acc[2] = fr29_canon_pack(fr29_mul(wide29_redc(w2), fix));
    acc[1] = sub(sub(fr29_canon_pack(fr29_mul(wide29_redc(wx), fix)), acc[0]), acc[2]);
    acc[3] = sum9_residue(sa0);
    acc[4] = sub(sum9_residue(sa1), acc[3]);
    block_reduce_store<5>(acc, partials);
}

// k_lookup_round<false, true> for queries given by their int32 forms (HintSrc::hint_ints), with the arithmetic of the common
// pair -- both inverses read from the table's records -- in 29-bit limbs: M = (a0 + a1)(s0 + s1') is one product, E M goes into
// an unreduced sum, the two folds are one product each; the sums of a0, of a1 and of E are plain 288-bit integers.  A pair
// with an inverse of its own (a query that is no table entry, or -beta) takes the formulas of the other kernel in 32-bit limbs.
// Same inputs, same outputs (folded tensors canonical, the five sums with the factors that kernel leaves on them).  At most
// 512 pairs per lane (the unreduced sum holds 2^522): the launch site checks.
__global__ void __launch_bounds__(TPB) k_lookup_first29(Fr* __restrict__ partials, Fr* __restrict__ nA, Fr* __restrict__ nS, const Fr* __restrict__ E, const Fr beta, const Fr v_mont,
                                                        size_t n_out, Fr* __restrict__ nE, const HintSrc hs) {
    const Fr29 vq = fr29_mul(fr29_repack(v_mont), fr29_2_266());      // v 2^261
    const Fr29 b2 = fr29_repack(add(beta, beta));
    Wide29 wx = wide29_zero();                                         // sum of E M over the pairs of unit inverses, times 2^-5
    uint32_t se[9], sa0[9], sa1[9];                                    // sums of E (those pairs), of a0 and of a1 (every pair)
#pragma unroll
    for (int i = 0; i < 9; ++i) se[i] = sa0[i] = sa1[i] = 0;
    Fr c0s = big_zero<8>(), c1s = big_zero<8>(), c2s = big_zero<8>();  // the three weighted terms of the other pairs
    uint32_t it = 0;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        const Fr e = ld_stream(E + t);
        if (nE && t < n_out / 2) st_stream(nE + t, add(e, ld_stream(E + t + n_out / 2)));      // the next round's table: the top variable summed out
        Fr s0w, s1w, a0w, a1w;
        bool unit0 = false, unit1 = false;
        s0w = query_inv_ints(t, hs, a0w, unit0);
        s1w = query_inv_ints(t + n_out, hs, a1w, unit1);
        sum9_add(sa0, a0w);
        sum9_add(sa1, a1w);
        if (unit0 && unit1) {
            const Fr29 a0 = fr29_repack(a0w), a1 = fr29_repack(a1w), s0 = fr29_repack(s0w), s1 = fr29_repack(s1w);
            sum9_add(se, e);
            const Fr29 M = fr29_mul(fr29_add(a0, a1), fr29_add(fr29_add(s0, s1), b2));
            wide29_mac(wx, fr29_repack(e), M);
            if ((++it & 3u) == 0u) wide29_carry(wx);
            st_stream(nA + t, fr29_canon_pack(fr29_add(a0, fr29_mul(vq, fr29_sub_plus_r(a1, a0)))));
            st_stream(nS + t, fr29_canon_pack(fr29_add(s0, fr29_mul(vq, fr29_sub_plus_r(s1, s0)))));
        } else {
            const Fr da = sub(a1w, a0w), ds = sub(s1w, s0w), s0 = add(s0w, beta);
            const Fr ea0 = mont_mul(e, a0w), eda = mont_mul(e, da);
            const Fr c0 = mont_mul(ea0, s0), c2 = mont_mul(eda, ds);
            c0s = add(c0s, c0);
            c1s = add(c1s, sub(sub(mont_mul(add(ea0, eda), add(s0, ds)), c0), c2));
            c2s = add(c2s, c2);
            st_stream(nA + t, add(a0w, mont_mul(v_mont, da)));
            st_stream(nS + t, add(s0w, mont_mul(v_mont, ds)));
        }
    }
    Fr acc[5];
    // E M 2^-5 summed; reduced (2^-261) and brought to the factor 2^-256 of the other kernel's products by 2^271 (2^-261 again)
    const Fr acc_em = fr29_canon_pack(fr29_mul(wide29_redc(wx), fr29_2_271()));
    // E is in Montgomery form and the sums carry R^-1: sum(E) R^-2 through one product with R^-1
    constexpr uint32_t RINV[8] = {4269129792u, 334977897u, 165441631u, 2876230287u, 1333208682u, 1912866698u, 805346647u, 465471123u};
    Fr k;
#pragma unroll
    for (int l = 0; l < 8; ++l) k.v[l] = RINV[l];
    const Fr one = mont_mul(sum9_residue(se), k), two = add(one, one), four = add(two, two);
    acc[0] = add(c0s, one);
    acc[1] = add(c1s, sub(acc_em, four));
    acc[2] = add(c2s, sub(four, acc_em));
    acc[3] = sum9_residue(sa0);
    acc[4] = sub(sum9_residue(sa1), acc[3]);
    block_reduce_store<5>(acc, partials);
}

// The first TWO rounds of such a job in one pass: the folded tensors of the first round are never written or read back.
// Lane t < h2 (h2 = a quarter of the queries) takes the quad t, t + h2, t + h1, t + h1 + h2 (h1 = 2 h2): the first round's pairs
// (t, t + h1) and (t + h2, t + h1 + h2) with their eq weights E[t], E[t + h2], exactly as k_lookup_first29 treats a pair; their
// folds by v1 are the second round's pair (t, t + h2), whose weight is the sum of the two (the top variable summed out), treated
// as k_lookup_round29 treats a pair except that its three weighted products are reduced one by one (three unreduced sums more
// would not fit two waves per SIMD, and this kernel is bound by its traffic: 176 bytes per quad instead of 528).  The second
// round's plain sums follow from four sums of the gathered inverses, one per quarter: sum a' = S_0 + v1 (S_1 - S_0).
// Writes the second round's folded tensors (h2 each), the third round's eq table (h2 / 2 entries) and both rounds' five sums
// (partials: round 1 at [0, 5 gridDim), round 2 behind it).  At most 256 quads per lane; the launch site checks.
// what every lane needs of the challenges, made on the host so that it arrives in scalar registers
// v 2^58 and its negative in 29-bit limbs (for fr29_mul_small): what a fold by v of two small integers multiplies by
struct SmallFold { Fr29 vs, nvs; };
static SmallFold small_fold_consts(const Fr& v_mont) {
    SmallFold c;
    Fr29 two63 = fr29_zero();
    two63.l[2] = 32;                                                    // 2^63: v 2^256 2^63 2^-261 = v 2^58
    c.vs = fr29_mul(fr29_repack(v_mont), two63);
    c.nvs = fr29_sub_plus_r(fr29_r(), c.vs);                            // 2 r - v 2^58: non-negative (the product is below 2 r)
    return c;
}
// x0 + v (x1 - x0) for 32-bit integers, canonical: one small-operand product
__device__ __forceinline__ Fr fold_small(int64_t x0, int64_t d, const SmallFold& c) {
    const bool ng = d < 0;
    const uint64_t k = ng ? 0ull - (uint64_t)d : (uint64_t)d;
    return fr29_canon_pack(fr29_add(fr29_from_small(x0), fr29_mul_small(ng ? c.nvs : c.vs, (uint32_t)k & R29M, (uint32_t)(k >> 29))));
}
// v1 2^261, v2 2^261, beta, 2 beta, 2^261 mod r (a product with it leaves the value, reduced); v1 2^58 and its negative (for
// fr29_mul_small: the first fold of a plain table's queries, which differ by a small integer)
struct First2Consts { Fr29 vq1, vq2, b29, b2, c261, vs1, nvs1; };
static First2Consts first2_consts(const Fr& beta, const Fr& v1_mont, const Fr& v2_mont) {
    First2Consts c;
    c.vq1 = fr29_mul(fr29_repack(v1_mont), fr29_2_266());
    c.vq2 = fr29_mul(fr29_repack(v2_mont), fr29_2_266());
    c.b29 = fr29_repack(beta);
    c.b2 = fr29_repack(add(beta, beta));
    Fr29 one29 = fr29_zero();
    one29.l[0] = 1;
    c.c261 = fr29_mul(fr29_2_522(), one29);
    const SmallFold sf = small_fold_consts(v1_mont);
    c.vs1 = sf.vs;
    c.nvs1 = sf.nvs;
    return c;
}
template <bool PLAIN> __global__ void __launch_bounds__(TPB) k_lookup_first2_29(Fr* __restrict__ partials, Fr* __restrict__ nA, Fr* __restrict__ nS, const Fr* __restrict__ E, const Fr beta,
                                                          const Fr v1_mont, const First2Consts cs, size_t h2, Fr* __restrict__ nE3, const HintSrc hs) {
    __shared__ uint32_t rare[3][8][TPB];                               // round 1: the three weighted terms of the pairs with an inverse of their own, per lane
    const size_t h1 = 2 * h2;
    const Fr29 vq1 = cs.vq1, vq2 = cs.vq2, b29 = cs.b29, b2 = cs.b2, c261 = cs.c261;
    // A plain table (no mapped values): two queries that are table entries differ by the small integer d = q1 - q0, and with
    // a0 (s0 + beta) = a1 (s1 + beta) = 1 (as Montgomery products) the pair's M - 4 is (a0 - a1) d (as a Montgomery product).  That product and the fold v1 d are small-operand
    // products (fr29_mul_small); wx then sums E (M - 4) 2^-58 instead of E M.
    constexpr bool plain = PLAIN;                                      // the launch site: hs.sout_ints == nullptr
    Wide29 wx = wide29_zero();                                         // round 1: sum of E M over the pairs of unit inverses, times 2^-5
    __shared__ uint32_t qsum[4][9][TPB];                               // sums of the inverses of the four quarters, per lane (registers are short here)
    uint32_t se[9];                                                    // sum of E over the pairs of unit inverses
#pragma unroll
    for (int i = 0; i < 9; ++i) se[i] = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int l = 0; l < 9; ++l) qsum[k][l][threadIdx.x] = 0;
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int l = 0; l < 8; ++l) rare[k][l][threadIdx.x] = 0;
    auto qsum_add = [&](int k, const Fr& x) {
        uint32_t acc[9];
#pragma unroll
        for (int l = 0; l < 9; ++l) acc[l] = qsum[k][l][threadIdx.x];
        sum9_add(acc, x);
#pragma unroll
        for (int l = 0; l < 9; ++l) qsum[k][l][threadIdx.x] = acc[l];
    };
    auto qsum_residue = [&](int k) {
        uint32_t acc[9];
#pragma unroll
        for (int l = 0; l < 9; ++l) acc[l] = qsum[k][l][threadIdx.x];
        return sum9_residue(acc);
    };
    Fr29 t0 = fr29_zero(), t2 = fr29_zero(), tx = fr29_zero();         // round 2: the three weighted sums, times 2^-266
    uint32_t it = 0;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < h2; t += (size_t)gridDim.x * TPB) {
        const Fr eA = ld_stream(E + t), eB = ld_stream(E + t + h2);
        if (nE3 && t < h2 / 2) st_stream(nE3 + t, add(add(eA, eB), add(ld_stream(E + t + h2 / 2), ld_stream(E + t + h2 + h2 / 2))));      // two variables summed out
        // the first round's folds: the second round's pair (named variables: an array indexed by the half would live in private memory)
        Fr29 fa0, fs0, fa1, fs1;
        auto first_round_pair = [&](size_t i, const Fr& e, int qa, int qb, Fr29& fa, Fr29& fs) {
            Fr s0w, s1w, a0w, a1w;
            bool unit0 = false, unit1 = false;
            int32_t q0 = 0, q1 = 0;
            s0w = query_inv_ints(i, hs, a0w, unit0, &q0);
            s1w = query_inv_ints(i + h1, hs, a1w, unit1, &q1);
            qsum_add(qa, a0w);
            qsum_add(qb, a1w);
            if constexpr (PLAIN) { if (unit0 && unit1) {
                const Fr29 a0 = fr29_repack(a0w), a1 = fr29_repack(a1w), s0 = fr29_repack(s0w);
                sum9_add(se, e);
                const int64_t d = (int64_t)q1 - (int64_t)q0;
                const bool ng = d < 0;
                const uint64_t k = ng ? 0ull - (uint64_t)d : (uint64_t)d;       // below 2^32
                const uint32_t k0 = (uint32_t)k & R29M, k1 = (uint32_t)(k >> 29);
                const Fr29 da = fr29_sub_plus_r(a1, a0), nda = fr29_sub_plus_r(a0, a1);
                wide29_mac(wx, fr29_repack(e), fr29_mul_small(ng ? da : nda, k0, k1));      // (a0 - a1) d 2^-58
                fa = fr29_add(a0, fr29_mul(vq1, da));
                fs = fr29_add(s0, fr29_mul_small(ng ? cs.nvs1 : cs.vs1, k0, k1));        // s0 + v1 d
                return;
            } }
            if (!PLAIN && unit0 && unit1) {
                const Fr29 a0 = fr29_repack(a0w), a1 = fr29_repack(a1w), s0 = fr29_repack(s0w), s1 = fr29_repack(s1w);
                sum9_add(se, e);
                const Fr29 M = fr29_mul(fr29_add(a0, a1), fr29_add(fr29_add(s0, s1), b2));
                wide29_mac(wx, fr29_repack(e), M);
                fa = fr29_add(a0, fr29_mul(vq1, fr29_sub_plus_r(a1, a0)));
                fs = fr29_add(s0, fr29_mul(vq1, fr29_sub_plus_r(s1, s0)));
            } else {
                const Fr da = sub(a1w, a0w), ds = sub(s1w, s0w), s0 = add(s0w, beta);
                const Fr ea0 = mont_mul(e, a0w), eda = mont_mul(e, da);
                const Fr c0 = mont_mul(ea0, s0), c2 = mont_mul(eda, ds);
                const Fr c1 = sub(sub(mont_mul(add(ea0, eda), add(s0, ds)), c0), c2);
                Fr r0, r1, r2;
#pragma unroll
                for (int l = 0; l < 8; ++l) { r0.v[l] = rare[0][l][threadIdx.x]; r1.v[l] = rare[1][l][threadIdx.x]; r2.v[l] = rare[2][l][threadIdx.x]; }
                r0 = add(r0, c0); r1 = add(r1, c1); r2 = add(r2, c2);
#pragma unroll
                for (int l = 0; l < 8; ++l) { rare[0][l][threadIdx.x] = r0.v[l]; rare[1][l][threadIdx.x] = r1.v[l]; rare[2][l][threadIdx.x] = r2.v[l]; }
                fa = fr29_repack(add(a0w, mont_mul(v1_mont, da)));
                fs = fr29_repack(add(s0w, mont_mul(v1_mont, ds)));
            }
        };
        first_round_pair(t, eA, 0, 2, fa0, fs0);              // quarters: 0 = [0, h2), 1 = [h2, h1), 2 = [h1, h1 + h2), 3 = the last
        first_round_pair(t + h2, eB, 1, 3, fa1, fs1);
        if ((++it & 1u) == 0u) wide29_carry(wx);                       // two terms a quad: a carry pass every fourth term
        // the second round over (fa0, fa1), (fs0, fs1); the folds are below 2.03 r, differences are taken with 3 r added
        const Fr29 e2 = fr29_add(fr29_repack(eA), fr29_repack(eB));
        const Fr29 da = fr29_sub_plus_3r(fa1, fa0), ds = fr29_sub_plus_3r(fs1, fs0);
        const Fr29 s0 = fr29_add(fs0, b29);
        const Fr29 ea0 = fr29_mul(e2, fa0), eda = fr29_mul(e2, da);
        t0 = fr29_add(t0, fr29_mul(ea0, s0));
        t2 = fr29_add(t2, fr29_mul(eda, ds));
        tx = fr29_add(tx, fr29_mul(fr29_add(ea0, eda), fr29_add(s0, ds)));
        if ((it & 31u) == 0u) { t0 = fr29_mul(t0, c261); t2 = fr29_mul(t2, c261); tx = fr29_mul(tx, c261); }      // the top limbs stay below 2^30
        st_stream(nA + t, fr29_canon_pack<3>(fr29_add(fa0, fr29_mul(vq2, da))));
        st_stream(nS + t, fr29_canon_pack<3>(fr29_add(fs0, fr29_mul(vq2, ds))));
    }
    const Fr29 fix = fr29_2_271();
    // round 1
    {
        Fr acc[5];
        Fr29 em29 = fr29_mul(wide29_redc(wx), fix);
        if (plain) {
            // The inverses are inverses under the Montgomery product, a (s + beta) = 2^256, and M is such a product:
            // M - 4 = (a0 - a1) d 2^-261 in this file's 29-bit form.  The small products left 2^-58: 2^-203 is missing.
            Fr29 two58 = fr29_zero();
            two58.l[2] = 1;
            em29 = fr29_mul(em29, two58);
        }
        const Fr acc_em = fr29_canon_pack(em29);
        constexpr uint32_t RINV[8] = {4269129792u, 334977897u, 165441631u, 2876230287u, 1333208682u, 1912866698u, 805346647u, 465471123u};
        Fr k;
#pragma unroll
        for (int l = 0; l < 8; ++l) k.v[l] = RINV[l];
        const Fr one = mont_mul(sum9_residue(se), k), two = add(one, one), four = plain ? big_zero<8>() : add(two, two);      // plain: acc_em is the sum of E (M - 4) already
        Fr c0s, c1s, c2s;
#pragma unroll
        for (int l = 0; l < 8; ++l) { c0s.v[l] = rare[0][l][threadIdx.x]; c1s.v[l] = rare[1][l][threadIdx.x]; c2s.v[l] = rare[2][l][threadIdx.x]; }
        acc[0] = add(c0s, one);
        acc[1] = add(c1s, sub(acc_em, four));
        acc[2] = add(c2s, sub(four, acc_em));
        acc[3] = add(qsum_residue(0), qsum_residue(1));
        acc[4] = sub(add(qsum_residue(2), qsum_residue(3)), acc[3]);
        block_reduce_store<5>(acc, partials);
    }
    // round 2
    {
        Fr acc[5];
        acc[0] = fr29_canon_pack(fr29_mul(t0, fix));
        acc[2] = fr29_canon_pack(fr29_mul(t2, fix));
        acc[1] = sub(sub(fr29_canon_pack(fr29_mul(tx, fix)), acc[0]), acc[2]);
        const Fr r00 = qsum_residue(0), r01 = qsum_residue(1);
        const Fr sA = add(r00, mont_mul(v1_mont, sub(qsum_residue(2), r00)));      // sum of fa0 over the lane's quads
        const Fr sB = add(r01, mont_mul(v1_mont, sub(qsum_residue(3), r01)));      // sum of fa1
        acc[3] = sA;
        acc[4] = sub(sB, sA);
        block_reduce_store<5>(acc, partials + 5 * (size_t)gridDim.x);
    }
}

// ---- Hadamard-product sumcheck with adjacent-pair folding (Fr_hp_sc, proof.cu:66-98) -------------------------------------
// One round over pairs (2g, 2g+1), zero beyond in_size: the three term tensors of the reference's step kernel
//   o0 = a0 b0,  o1 = a0 db + b0 da,  o2 = da db      (each product carries R^-1: the reference multiplies standard-form
//                                                      values with the Montgomery routine and does not convert back)
// are never written: their multilinear evaluations at the remaining challenges, sum_g eq[g] o_k[g], are accumulated
// directly (E in Montgomery form, so E * o is a plain product), a and b are folded by v, and the eq table of the next
// round (this round's lowest variable summed out) is written on the way.
__global__ void __launch_bounds__(TPB) k_hp_round(Fr* __restrict__ partials, Fr* __restrict__ nA, Fr* __restrict__ nB, Fr* __restrict__ nE, const Fr* __restrict__ A,
                                                  const Fr* __restrict__ B, const Fr* __restrict__ E, const Fr v_mont, size_t in_size, size_t out_size, size_t ne_count) {
    Fr acc[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) acc[i] = big_zero<8>();
    for (size_t g = (size_t)blockIdx.x * TPB + threadIdx.x; g < out_size; g += (size_t)gridDim.x * TPB) {
        const Fr a0 = A[2 * g], b0 = B[2 * g];
        const Fr a1 = (2 * g + 1 < in_size) ? A[2 * g + 1] : big_zero<8>(), b1 = (2 * g + 1 < in_size) ? B[2 * g + 1] : big_zero<8>();
        const Fr da = sub(a1, a0), db = sub(b1, b0);
        const Fr e = E[g];
        // the eq weight on one factor first: five products instead of seven (a0 db + b0 da = (a0 + da)(b0 + db) - a0 b0 - da db)
        const Fr ea0 = mont_mul(e, a0), eda = mont_mul(e, da);
        const Fr c0 = mont_mul(ea0, b0), c2 = mont_mul(eda, db);
        acc[0] = add(acc[0], c0);
        acc[1] = add(acc[1], sub(sub(mont_mul(add(ea0, eda), add(b0, db)), c0), c2));
        acc[2] = add(acc[2], c2);
        nA[g] = add(a0, mont_mul(v_mont, da));
        nB[g] = add(b0, mont_mul(v_mont, db));
        if (g < ne_count) nE[g] = add(E[2 * g], E[2 * g + 1]);
    }
    block_reduce_store<3>(acc, partials);
}

// ---- multi-Hadamard sumcheck round (proof.cu:191-241) --------------------------------------------------------------------------
// K tensors; coefficient j of prod_k (X0_k + t dX_k), weighted by E and summed (R^-K attached... see host);
// also folds every tensor by v.
template <int K> struct PtrPack { const Fr* in[K]; Fr* out[K]; };
template <int K> __global__ void __launch_bounds__(TPB)
k_hadamard_round(Fr* __restrict__ partials, const PtrPack<K> p, const Fr* __restrict__ E, const Fr v_mont, size_t n_out, Fr* __restrict__ nE) {
    Fr acc[K + 1];
#pragma unroll
    for (int i = 0; i <= K; ++i) acc[i] = big_zero<8>();
    WideAcc w0 = wide_zero(), w2 = wide_zero(), wx = wide_zero();      // K == 2: sums of E x0 y0, E dx dy and E x1 y1
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        // Coefficients of the running product from standard-form values: every coefficient is a sum of products of the same
        // number of factors, so each Montgomery product leaves one more R^-1 on all of them alike (K - 1 in the end), which
        // the lane's sums shed once after the loop instead of every value being converted before it is multiplied.
        Fr c[K + 1];
        if constexpr (K == 2) {
            const Fr x0 = p.in[0][t], x1 = p.in[0][t + n_out], y0 = p.in[1][t], y1 = p.in[1][t + n_out];
            const Fr dx = sub(x1, x0), dy = sub(y1, y0);
            p.out[0][t] = add(x0, mont_mul(v_mont, dx));
            p.out[1][t] = add(y0, mont_mul(v_mont, dy));
            // E goes onto x0 and dx first (e is loaded below for the other K): the three weighted coefficients cost five
            // products instead of six.  x0 dy + y0 dx = x1 y1 - x0 y0 - dx dy.
            const Fr e2 = E[t];
            const Fr ex0 = mont_mul(e2, x0), edx = mont_mul(e2, dx);
            // the three products are summed unreduced (one reduction per lane after the loop); c stays zero
            wide_mac(w0, ex0, y0);
            wide_mac(w2, edx, dy);
            wide_mac(wx, add(ex0, edx), y1);
            c[0] = c[1] = c[2] = big_zero<8>();
        } else {
            {
                const Fr x0 = p.in[0][t], x1 = p.in[0][t + n_out];
                const Fr dx = sub(x1, x0);
                const Fr e1 = E[t];
                c[0] = mont_mul(e1, x0); c[1] = mont_mul(e1, dx);       // the weight first: no product with E per coefficient later
                p.out[0][t] = add(x0, mont_mul(v_mont, dx));
            }
#pragma unroll
            for (int k = 1; k < K; ++k) {
                const Fr x0 = p.in[k][t], x1 = p.in[k][t + n_out];
                const Fr dx = sub(x1, x0);
                p.out[k][t] = add(x0, mont_mul(v_mont, dx));
                c[k + 1] = mont_mul(c[k], dx);
#pragma unroll
                for (int j = k; j >= 1; --j) c[j] = add(mont_mul(c[j], x0), mont_mul(c[j - 1], dx));
                c[0] = mont_mul(c[0], x0);
            }
        }
        const Fr e = E[t];   // Montgomery form: e*R
        if (nE && t < n_out / 2) nE[t] = add(e, E[t + n_out / 2]);      // the next round's table
        if constexpr (K != 2) {
#pragma unroll
            for (int j = 0; j <= K; ++j) acc[j] = add(acc[j], c[j]);
        }
    }
    if constexpr (K == 2) {
        acc[0] = wide_redc(w0);
        acc[2] = wide_redc(w2);
        acc[1] = sub(sub(wide_redc(wx), acc[0]), acc[2]);
    }
    if (K > 1) {
        const Fr r2 = big_r2<8>();
#pragma unroll
        for (int j = 0; j <= K; ++j)
#pragma unroll
            for (int f = 1; f < K; ++f) acc[j] = mont_mul(acc[j], r2);
    }
    block_reduce_store<K + 1>(acc, partials);
}

// k_hadamard_round<2> for rounds of many pairs with the arithmetic in 29-bit limbs, as k_lookup_round29 does it: the weight
// arrives as E 2^256, e x0 and e dx come out as E x0 / 32 and E dx / 32, the three sums of products stay unreduced, are
// reduced once per lane (2^-261 again) and brought to standard form by 2^271 (2^-261 once more: R^-1 in all) and R^2.
// Same inputs, same outputs (folded tensors canonical).  At most 256 pairs per lane: the launch site checks.
__global__ void __launch_bounds__(TPB) k_hadamard_round29(Fr* __restrict__ partials, Fr* __restrict__ nX, Fr* __restrict__ nY, const Fr* __restrict__ X, const Fr* __restrict__ Y,
                                                          const Fr* __restrict__ E, const Fr v_mont, size_t n_out, Fr* __restrict__ nE) {
    const Fr29 vq = fr29_mul(fr29_repack(v_mont), fr29_2_266());      // v 2^261
    Wide29 w0 = wide29_zero(), w2 = wide29_zero(), wx = wide29_zero();
    uint32_t it = 0;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        const Fr e = E[t];
        if (nE && t < n_out / 2) nE[t] = add(e, E[t + n_out / 2]);      // the next round's table: the top variable summed out
        const Fr29 x0 = fr29_repack(X[t]), y0 = fr29_repack(Y[t]), y1 = fr29_repack(Y[t + n_out]);
        const Fr29 dx = fr29_sub_plus_r(fr29_repack(X[t + n_out]), x0), dy = fr29_sub_plus_r(y1, y0);      // + r: non-negative, the same residues
        const Fr29 e29 = fr29_repack(e);
        const Fr29 ex0 = fr29_mul(e29, x0), edx = fr29_mul(e29, dx);
        wide29_mac(w0, ex0, y0);
        wide29_mac(w2, edx, dy);
        wide29_mac(wx, fr29_add(ex0, edx), y1);                          // x0 dy + y0 dx = x1 y1 - x0 y0 - dx dy
        if ((++it & 3u) == 0u) { wide29_carry(w0); wide29_carry(w2); wide29_carry(wx); }
        nX[t] = fr29_canon_pack(fr29_add(x0, fr29_mul(vq, dx)));
        nY[t] = fr29_canon_pack(fr29_add(y0, fr29_mul(vq, dy)));
    }
    Fr acc[3];
    const Fr29 fix = fr29_2_271();
    acc[0] = fr29_canon_pack(fr29_mul(wide29_redc(w0), fix));
    acc[2] = fr29_canon_pack(fr29_mul(wide29_redc(w2), fix));
    acc[1] = sub(sub(fr29_canon_pack(fr29_mul(wide29_redc(wx), fix)), acc[0]), acc[2]);
    const Fr r2 = big_r2<8>();
#pragma unroll
    for (int j = 0; j < 3; ++j) acc[j] = mont_mul(acc[j], r2);
    block_reduce_store<3>(acc, partials);
}

// The first round for two tensors given by their int32 forms (the mapped outputs of a softmax's segments): 4 bytes per
// element instead of 32, and the three weighted coefficients are E times an exact 64-bit integer (x0 y0, dx dy, x1 y1) --
// sixteen limb products into an unreduced twelve-limb sum each, one reduction per lane -- instead of Montgomery products.
// The sums come out as k_hadamard_round<2> leaves them (standard form, no factor of R).
__device__ __forceinline__ void imac64(uint32_t (&acc)[12], const Fr& e, const Fr& ne, int64_t a, int64_t b) {
    const uint64_t ma = a < 0 ? 0ull - (uint64_t)a : (uint64_t)a, mb = b < 0 ? 0ull - (uint64_t)b : (uint64_t)b;      // both below 2^32
    const uint64_t mag = ma * mb;
    const bool ng = (a < 0) != (b < 0);
    const uint32_t m0 = (uint32_t)mag, m1 = (uint32_t)(mag >> 32);
    uint32_t s[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = ng ? ne.v[i] : e.v[i];
    uint64_t carry = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint64_t t = (uint64_t)s[i] * m0 + acc[i] + carry;
        acc[i] = (uint32_t)t;
        carry = t >> 32;
    }
#pragma unroll
    for (int i = 8; i < 12; ++i) {
        const uint64_t t = (uint64_t)acc[i] + carry;
        acc[i] = (uint32_t)t;
        carry = t >> 32;
    }
    carry = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint64_t t = (uint64_t)s[i] * m1 + acc[i + 1] + carry;
        acc[i + 1] = (uint32_t)t;
        carry = t >> 32;
    }
#pragma unroll
    for (int i = 9; i < 12; ++i) {
        const uint64_t t = (uint64_t)acc[i] + carry;
        acc[i] = (uint32_t)t;
        carry = t >> 32;
    }
}
__device__ __forceinline__ Fr imac64_finish(const uint32_t (&acc)[12]) {
    Fr lo, hi = big_zero<8>(), one = big_zero<8>();
#pragma unroll
    for (int i = 0; i < 8; ++i) lo.v[i] = acc[i];
    lo = reduce_once(reduce_once(lo));
    one.v[0] = 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) hi.v[i] = acc[8 + i];
    return add(mont_mul(lo, one), hi);
}
__global__ void __launch_bounds__(TPB) k_hadamard_round2_ints(Fr* __restrict__ partials, const int32_t* __restrict__ X, const int32_t* __restrict__ Y, Fr* __restrict__ outx,
                                                              Fr* __restrict__ outy, const Fr* __restrict__ E, const SmallFold vc, size_t n_out, Fr* __restrict__ nE) {
    uint32_t a0[12], a2[12], ax[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) a0[i] = a2[i] = ax[i] = 0;
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) {
        const int64_t x0 = X[t], x1 = X[t + n_out], y0 = Y[t], y1 = Y[t + n_out];
        const int64_t dx = x1 - x0, dy = y1 - y0;
        outx[t] = fold_small(x0, dx, vc);
        outy[t] = fold_small(y0, dy, vc);
        const Fr e = E[t];
        const Fr ne = neg(e);
        if (nE && t < n_out / 2) nE[t] = add(e, E[t + n_out / 2]);
        imac64(a0, e, ne, x0, y0);
        imac64(a2, e, ne, dx, dy);
        imac64(ax, e, ne, x1, y1);
    }
    Fr acc[3];
    acc[0] = imac64_finish(a0);
    acc[2] = imac64_finish(a2);
    acc[1] = sub(sub(imac64_finish(ax), acc[0]), acc[2]);
    block_reduce_store<3>(acc, partials);
}

// ---- the last rounds of a sumcheck in one launch ---------------------------------------------------------------------------------
// Once the tensors are short, a round is a few microseconds of arithmetic between two host round trips.  The
// challenges of these sumchecks are fixed before the first round (tLookup::prove and multi_hadamard_sumchecks take u and
// v as arguments, tlookup.cu:150-176, proof.cu:191-241), so one workgroup can run every remaining round back to back --
// sums, fold by v, halving of the eq table, workgroup barrier -- and hand all rounds' sums back in one copy.
static constexpr int TAIL_T = 1024;          // lanes of the single workgroup
static constexpr int TAIL_HALF = 256;        // largest n_out of the first fused round: one compute unit does all of it
static constexpr int TAIL_ROUNDS = 16;
struct TailV { Fr v[TAIL_ROUNDS]; };         // Montgomery form, in round order
static constexpr int SPLIT_HALF = 32768;     // rounds of at most this many pairs spread each pair over several lanes

__device__ __forceinline__ Fr wave_sum(Fr x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Fr y;
#pragma unroll
        for (int l = 0; l < 8; ++l) y.v[l] = __shfl_down(x.v[l], off, 64);
        x = add(x, y);
    }
    return x;
}
// sums of K values over the TAIL_T lanes into out[0..K) (lane 0 writes); red: K x 16 x 8 words of LDS
template <int K> __device__ __forceinline__ void tail_block_sum(Fr (&acc)[K], Fr* __restrict__ out, uint32_t* red) {
    const uint32_t t = threadIdx.x, wv = t >> 6, ln = t & 63u;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const Fr w = wave_sum(acc[k]);
        if (ln == 0) {
#pragma unroll
            for (int l = 0; l < 8; ++l) red[(k * 16 + wv) * 8 + l] = w.v[l];
        }
    }
    __syncthreads();
    if (wv == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            Fr x = big_zero<8>();
            if (ln < 16) {
#pragma unroll
                for (int l = 0; l < 8; ++l) x.v[l] = red[(k * 16 + ln) * 8 + l];
            }
            x = wave_sum(x);
            if (ln == 0) out[k] = x;
        }
    }
    __syncthreads();
}

// A lookup round splits into four independent tasks per pair, so that short rounds -- where lanes are plentiful and the
// chain of ~20 dependent field multiplications per pair is what takes the time -- can spread a pair over four lanes:
//   task 0: sums 0..2 (E-weighted products of A and S + beta)        task 1: sums 5..7 (the same for B and T + beta)
//   task 2: sums 8..10 (products of m and B), folds of m, A and S     task 3: sums 3..4 (a0, da), folds of B and T
// Phase 1 has tasks 0 and 3' only (3' = sums 3..4 and the folds of A and S).  acc receives the task's sums (up to 3).
struct LookupPtrs {
    const Fr *A, *S, *B, *T, *m, *E;
    Fr *nA, *nS, *nB, *nT, *nm;
    Fr* nE;      // the next round's eq table (the top variable summed out), written by task 3; may be null
};
__device__ __forceinline__ void lookup_task(Fr (&acc)[3], int task, bool phase2, const LookupPtrs& p, const Fr& beta, const Fr& v_mont, size_t t, size_t n_out) {
    if (task == 0) {
        const Fr e = p.E[t];
        const Fr a0 = p.A[t], a1 = p.A[t + n_out], s0r = p.S[t], s1 = p.S[t + n_out];
        const Fr da = sub(a1, a0), ds = sub(s1, s0r), s0 = add(s0r, beta);
        acc[0] = add(acc[0], mont_mul(e, mont_mul(a0, s0)));
        acc[1] = add(acc[1], mont_mul(e, add(mont_mul(da, s0), mont_mul(a0, ds))));
        acc[2] = add(acc[2], mont_mul(e, mont_mul(da, ds)));
    } else if (task == 1) {
        const Fr e = p.E[t];
        const Fr b0 = p.B[t], b1 = p.B[t + n_out], t0r = p.T[t], t1 = p.T[t + n_out];
        const Fr db = sub(b1, b0), dt = sub(t1, t0r), t0 = add(t0r, beta);
        acc[0] = add(acc[0], mont_mul(e, mont_mul(b0, t0)));
        acc[1] = add(acc[1], mont_mul(e, add(mont_mul(db, t0), mont_mul(b0, dt))));
        acc[2] = add(acc[2], mont_mul(e, mont_mul(db, dt)));
    } else if (task == 2) {
        const Fr b0 = p.B[t], b1 = p.B[t + n_out], m0 = p.m[t], m1 = p.m[t + n_out];
        const Fr db = sub(b1, b0), dm = sub(m1, m0);
        acc[0] = add(acc[0], mont_mul(m0, b0));
        acc[1] = add(acc[1], add(mont_mul(dm, b0), mont_mul(m0, db)));
        acc[2] = add(acc[2], mont_mul(dm, db));
        p.nm[t] = add(m0, mont_mul(v_mont, dm));
        const Fr a0 = p.A[t], s0 = p.S[t];
        p.nA[t] = add(a0, mont_mul(v_mont, sub(p.A[t + n_out], a0)));
        p.nS[t] = add(s0, mont_mul(v_mont, sub(p.S[t + n_out], s0)));
    } else {
        if (p.nE && t < n_out / 2) p.nE[t] = add(p.E[t], p.E[t + n_out / 2]);
        const Fr a0 = p.A[t];
        const Fr da = sub(p.A[t + n_out], a0);
        acc[0] = add(acc[0], a0);
        acc[1] = add(acc[1], da);
        if (phase2) {
            const Fr b0 = p.B[t], t0 = p.T[t];
            p.nB[t] = add(b0, mont_mul(v_mont, sub(p.B[t + n_out], b0)));
            p.nT[t] = add(t0, mont_mul(v_mont, sub(p.T[t + n_out], t0)));
        } else {
            const Fr s0 = p.S[t];
            p.nA[t] = add(a0, mont_mul(v_mont, da));
            p.nS[t] = add(s0, mont_mul(v_mont, sub(p.S[t + n_out], s0)));
        }
    }
}
// where a task's sums go in the 11-value layout of a round, and how many it has
__device__ __forceinline__ int lookup_task_base(int task) { return task == 0 ? 0 : (task == 1 ? 5 : (task == 2 ? 8 : 3)); }
__device__ __forceinline__ int lookup_task_count(int task) { return task == 3 ? 2 : 3; }

// One round, one task per blockIdx.y (phase 1: y = 0 -> task 0, y = 1 -> task 3; phase 2: y = task).
// partials[k * gridDim.x + blockIdx.x] for the sums k the task owns.
template <bool PHASE2> __global__ void __launch_bounds__(TPB)
k_lookup_round_split(Fr* __restrict__ partials, const LookupPtrs p, const Fr beta, const Fr v_mont, size_t n_out) {
    const int task = PHASE2 ? (int)blockIdx.y : (blockIdx.y == 0 ? 0 : 3);
    Fr acc[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) acc[i] = big_zero<8>();
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n_out; t += (size_t)gridDim.x * TPB) lookup_task(acc, task, PHASE2, p, beta, v_mont, t, n_out);
    if (task == 3) {                      // two sums only: row 5 belongs to task 1
        Fr a2[2] = {acc[0], acc[1]};
        block_reduce_store<2>(a2, partials + (size_t)3 * gridDim.x);
    } else {
        block_reduce_store<3>(acc, partials + (size_t)lookup_task_base(task) * gridDim.x);
    }
}

// All remaining rounds of the lookup sumcheck in one workgroup of four 256-lane groups, one per task.  Round r reads
// buffer set r & 1 and writes the other (round 0 reads the caller's tensors).  sums[r*11 + i] as k_lookup_round orders
// them (5 used in phase 1).  Rounds from `phase2_from` on are phase-2 rounds.  w: 2 x 6 x n_out0 elements of work space.
__global__ void __launch_bounds__(TAIL_T)
k_lookup_tail(Fr* __restrict__ sums, Fr* w, const Fr* A, const Fr* S, const Fr* B, const Fr* T, const Fr* m, const Fr* E,
              const Fr beta, const TailV vs, uint32_t n_out0, uint32_t rounds, uint32_t phase2_from) {
    __shared__ uint32_t red[4 * 3 * 4 * 8];       // task x sum x wave x limb
    const uint32_t grp = threadIdx.x >> 8, lt = threadIdx.x & 255u, wv = lt >> 6, ln = lt & 63u;
    LookupPtrs p;
    p.A = A; p.S = S; p.B = B; p.T = T; p.m = m; p.E = E; p.nE = nullptr;
    const Fr* cE = E;
    uint32_t n_out = n_out0;
    for (uint32_t r = 0; r < rounds; ++r) {
        const bool phase2 = r >= phase2_from;
        Fr* ws = w + (size_t)(r & 1u) * 6 * n_out0;
        p.nA = ws; p.nS = ws + n_out0; p.nB = ws + 2 * (size_t)n_out0; p.nT = ws + 3 * (size_t)n_out0; p.nm = ws + 4 * (size_t)n_out0;
        Fr* nE = ws + 5 * (size_t)n_out0;
        p.E = cE;
        const int task = (int)grp;
        const bool works = phase2 || task == 0 || task == 3;
        Fr acc[3];
#pragma unroll
        for (int i = 0; i < 3; ++i) acc[i] = big_zero<8>();
        if (works)
            for (uint32_t t = lt; t < n_out; t += 256) lookup_task(acc, task, phase2, p, beta, vs.v[r], t, n_out);
        // the halved eq table for the next round, by the lanes that idle in phase 1 (task 1) or finish early (any)
        const uint32_t nh = n_out >> 1;
        if (task == 1)
            for (uint32_t t = lt; t < nh; t += 256) nE[t] = add(cE[t], cE[t + nh]);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const Fr s = wave_sum(acc[k]);
            if (ln == 0) {
#pragma unroll
                for (int l = 0; l < 8; ++l) red[((grp * 3 + k) * 4 + wv) * 8 + l] = s.v[l];
            }
        }
        __syncthreads();
        if (wv == 0 && ln < 3 && (int)ln < lookup_task_count(task) && works) {
            Fr x = big_zero<8>();
            for (int q = 0; q < 4; ++q) {
                Fr y;
#pragma unroll
                for (int l = 0; l < 8; ++l) y.v[l] = red[((grp * 3 + ln) * 4 + q) * 8 + l];
                x = add(x, y);
            }
            sums[(size_t)r * 11 + lookup_task_base(task) + ln] = x;
        }
        p.A = p.nA; p.S = p.nS;
        if (phase2) { p.B = p.nB; p.T = p.nT; p.m = p.nm; }
        cE = nE;
        n_out = nh;
        __syncthreads();
    }
}

// All remaining rounds of the multi-Hadamard sumcheck for K tensors; sums[r*(K+1) + j].
template <int K> __global__ void __launch_bounds__(TAIL_T)
k_hadamard_tail(Fr* __restrict__ sums, const PtrPack<K> p, Fr* wE, const Fr* E, const TailV vs, uint32_t n_out0, uint32_t rounds) {
    __shared__ uint32_t red[(K + 1) * 16 * 8];
    const Fr* cur[K];
#pragma unroll
    for (int k = 0; k < K; ++k) cur[k] = p.in[k];
    const Fr* cE = E;
    const Fr r2 = big_r2<8>();
    uint32_t n_out = n_out0;
    for (uint32_t r = 0; r < rounds; ++r) {
        const Fr v_mont = vs.v[r];
        Fr acc[K + 1];
#pragma unroll
        for (int i = 0; i <= K; ++i) acc[i] = big_zero<8>();
        for (uint32_t t = threadIdx.x; t < n_out; t += TAIL_T) {
            Fr c[K + 1];
            {
                const Fr x0 = cur[0][t], x1 = cur[0][t + n_out];
                const Fr dx = sub(x1, x0);
                c[0] = x0; c[1] = dx;
                p.out[0][t] = add(x0, mont_mul(v_mont, dx));
            }
#pragma unroll
            for (int k = 1; k < K; ++k) {
                const Fr x0 = cur[k][t], x1 = cur[k][t + n_out];
                const Fr dx = sub(x1, x0);
                p.out[k][t] = add(x0, mont_mul(v_mont, dx));
                const Fr x0m = mont_mul(x0, r2), dxm = mont_mul(dx, r2);
                c[k + 1] = mont_mul(c[k], dxm);
#pragma unroll
                for (int j = k; j >= 1; --j) c[j] = add(mont_mul(c[j], x0m), mont_mul(c[j - 1], dxm));
                c[0] = mont_mul(c[0], x0m);
            }
            const Fr e = cE[t];
#pragma unroll
            for (int j = 0; j <= K; ++j) acc[j] = add(acc[j], mont_mul(e, c[j]));
        }
        tail_block_sum<K + 1>(acc, sums + (size_t)r * (K + 1), red);
#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = p.out[k];
        const uint32_t nh = n_out >> 1;
        for (uint32_t t = threadIdx.x; t < nh; t += TAIL_T) wE[t] = add(cE[t], cE[t + nh]);
        cE = wE;
        n_out = nh;
        __syncthreads();
    }
}

// ---- rescaling (rescaling.cu:8-21) ----------------------------------------------------------------------------------------------
// rem_ints (optional): the remainders once more as int32 (they lie in [-sf/2, sf/2))
// out_ints (optional): the rescaled values as int32 too; *flag is raised when one of them does not fit
__global__ void __launch_bounds__(TPB) k_rescale(Fr* __restrict__ out, Fr* __restrict__ rem, int32_t* __restrict__ rem_ints, const Fr* __restrict__ in, int64_t sf, size_t n,
                                                 int32_t* __restrict__ out_ints = nullptr, uint32_t* __restrict__ flag = nullptr) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int64_t hsf = sf >> 1;
    const int64_t x = fr_to_i64(in[i]);
    int64_t x_rem, x_rescaled;
    if ((sf & (sf - 1)) == 0) {          // a power of two (the same for every lane): the non-negative residue by mask, the exact quotient by shift
        x_rem = ((x + hsf) & (sf - 1)) - hsf;
        x_rescaled = (x - x_rem) >> (63 - __builtin_clzll((unsigned long long)sf));
    } else {
        const int64_t temp = (x + hsf) % sf;
        x_rem = (temp < 0 ? temp + sf : temp) - hsf;
        x_rescaled = (x - x_rem) / sf;
    }
    out[i] = fr_from_i64(x_rescaled);
    if (rem) rem[i] = fr_from_i64(x_rem);
    if (rem_ints) rem_ints[i] = (int32_t)x_rem;
    if (out_ints) {
        out_ints[i] = (int32_t)x_rescaled;
        if (x_rescaled != (int64_t)(int32_t)x_rescaled) atomicOr(flag, 1u);
    }
}
__global__ void __launch_bounds__(TPB) k_i32_fill(int32_t* __restrict__ dst, int32_t v, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) dst[i] = v;
}

// ---- ReLU decomposition (zkrelu.cu:8-29) -----------------------------------------------------------------------------------------
// The rescaling above, then the rescaled value split into sign (1 when >= 0), magnitude and max(., 0).
__global__ void __launch_bounds__(TPB) k_relu_decomp(Fr* __restrict__ res, Fr* __restrict__ sign, Fr* __restrict__ mag, Fr* __restrict__ rem,
                                                     const Fr* __restrict__ in, int64_t sf, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int64_t hsf = sf >> 1;
    const int64_t x = fr_to_i64(in[i]);
    const int64_t temp = (x + hsf) % sf;
    const int64_t x_rem = (temp < 0 ? temp + sf : temp) - hsf;
    const int64_t x_rescaled = (x - x_rem) / sf;
    const bool pos = x_rescaled >= 0;
    sign[i] = fr_from_u64(pos ? 1u : 0u);
    mag[i] = fr_from_i64(pos ? x_rescaled : -x_rescaled);
    rem[i] = fr_from_i64(x_rem);
    res[i] = pos ? fr_from_i64(x_rescaled) : big_zero<8>();
}

// ---- softmax (zksoftmax.cu) ------------------------------------------------------------------------------------------------------
// One wave per row.  The row's exponentials are added into ONE running sum in index order, as the one-thread-per-row
// loop of zksoftmax.cu:24-26 does: the 64 lanes evaluate 64 consecutive terms side by side, park them in LDS, and every
// lane then adds them in order (the additions are the same in all lanes, so all end with the same total).
// shift = round_half_away(scale * log(total)).  out = x - shift.  scale = sf_in * sqrt(d).
struct U32Pack8 { uint32_t v[8]; };
struct PlanePtrs { Fr* p[8]; };
struct IntPlanePtrs { int32_t* p[8]; };       // optional: the digits once more as int32 (a plane whose radix passes 2^31 gets none)
// digits of -x in the mixed radix bs[0..K) into position g of the planes (zksoftmax.cu:95-109)
__device__ __forceinline__ void softmax_digits(const PlanePtrs& planes, const IntPlanePtrs& ints, uint32_t* __restrict__ flag, const Fr& x, const U32Pack8& bs, int K, size_t g) {
    const Fr mx = neg(x);
    if (mx.v[2] | mx.v[3] | mx.v[4] | mx.v[5] | mx.v[6] | mx.v[7]) {
        atomicOr(flag, 1u);
        for (int k = 0; k < K; ++k) {
            if (planes.p[k]) planes.p[k][g] = big_zero<8>();
            if (ints.p[k]) ints.p[k][g] = 0;
        }
        return;
    }
    unsigned long long tmp = ((unsigned long long)mx.v[1] << 32) | mx.v[0];
    for (int k = 0; k < K; ++k) {
        const unsigned long long digit = tmp % bs.v[k];
        if (planes.p[k]) planes.p[k][g] = fr_from_u64(digit);
        if (ints.p[k]) ints.p[k][g] = (int32_t)digit;
        tmp /= bs.v[k];
    }
    if (tmp != 0) atomicOr(flag, 2u);   // more digits than the radices cover
}
// the same from the non-negative integer itself (negative: the shifted score was positive, the flag's first bit as above); a
// radix that is a power of two -- the same for every lane -- takes its digit by mask and shift instead of a 64-bit division
__device__ __forceinline__ void softmax_digits_u64(const PlanePtrs& planes, const IntPlanePtrs& ints, uint32_t* __restrict__ flag, bool negative, unsigned long long tmp,
                                                   const U32Pack8& bs, int K, size_t g) {
    if (negative) {
        atomicOr(flag, 1u);
        for (int k = 0; k < K; ++k) {
            if (planes.p[k]) planes.p[k][g] = big_zero<8>();
            if (ints.p[k]) ints.p[k][g] = 0;
        }
        return;
    }
    for (int k = 0; k < K; ++k) {
        const uint32_t b = bs.v[k];
        unsigned long long digit;
        if ((b & (b - 1u)) == 0u) {
            digit = tmp & (unsigned long long)(b - 1u);
            tmp >>= (31 - __builtin_clz(b));
        } else {
            digit = tmp % b;
            tmp /= b;
        }
        if (planes.p[k]) planes.p[k][g] = fr_from_u64(digit);
        if (ints.p[k]) ints.p[k][g] = (int32_t)digit;
    }
    if (tmp != 0) atomicOr(flag, 2u);   // more digits than the radices cover
}
static constexpr int SHIFT_ROW_CACHE = 2048;
// K > 0: the shifted scores are decomposed where they are written (k_softmax_decompose's planes without its pass over them)
// X64 set: the scores are given as 64-bit integers (a matrix product written in that form) and X is not read
__global__ void __launch_bounds__(TPB) k_softmax_shift(Fr* __restrict__ shift, Fr* __restrict__ out, const Fr* __restrict__ X, uint32_t rows, uint32_t cols, double scale,
                                                       const PlanePtrs planes, const IntPlanePtrs ints, uint32_t* __restrict__ flag, const U32Pack8 bs, int K,
                                                       const int64_t* __restrict__ X64 = nullptr) {
    __shared__ double term[TPB / 64][64];
    // Rows of up to SHIFT_ROW_CACHE scores are read once: the first pass leaves each score as a 64-bit integer in LDS and the
    // second takes it from there (a score that is no 64-bit integer raises the flag: its digits could not be formed either).
    __shared__ int64_t cache[TPB / 64][SHIFT_ROW_CACHE];
    const bool cached = flag != nullptr && cols <= (uint32_t)SHIFT_ROW_CACHE;      // (the plain shift has no flag to raise: it reads twice)
    const uint32_t w = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * (TPB / 64) + w;
    const bool live = row < rows;                         // a whole wave is live or idle; idle waves still reach every barrier
    const Fr* xr = X + (size_t)(live ? row : 0) * cols;
    const int64_t* xr64 = X64 ? X64 + (size_t)(live ? row : 0) * cols : nullptr;
    double total = 0.0;
    for (uint32_t j0 = 0; j0 < cols; j0 += 64) {
        const uint32_t j = j0 + lane;
        double tv = 0.0;
        if (live && j < cols) {
            int64_t xi;
            if (xr64) {
                xi = xr64[j];
                if (cached) cache[w][j] = xi;
            } else {
                const Fr x = xr[j];
                xi = fr_to_i64(x);
                if (cached) {
                    cache[w][j] = xi;
                    if (!equal(fr_from_i64(xi), x)) atomicOr(flag, 2u);
                }
            }
            tv = zkd::exp_det((double)xi / scale);
        }
        term[w][lane] = tv;
        __syncthreads();
        const uint32_t cnt = cols - j0 < 64u ? cols - j0 : 64u;
        if (cnt == 64u) {
#pragma unroll
            for (int q = 0; q < 64; ++q) total = total + term[w][q];
        } else {
            for (uint32_t q = 0; q < cnt; ++q) total = total + term[w][q];
        }
        __syncthreads();
    }
    if (!live) return;
    const double sv = scale * zkd::log_det(total);
    const int64_t si = (sv >= 0) ? (int64_t)(sv + 0.5) : (int64_t)(sv - 0.5);
    const Fr sh = fr_from_i64(si);
    if (lane == 0) shift[row] = sh;
    Fr* orow = out + (size_t)row * cols;
    for (uint32_t j = lane; j < cols; j += 64) {
        if (cached || xr64) {
            // the score as an integer: its shifted value and the digits of the negative from 64-bit arithmetic
            const int64_t xi = cached ? cache[w][j] : xr64[j];
            if (out) orow[j] = sub(fr_from_i64(xi), sh);
            const int64_t d = si - xi;
            if (K > 0) softmax_digits_u64(planes, ints, flag, d < 0, (unsigned long long)d, bs, K, (size_t)row * cols + j);
            continue;
        }
        const Fr xs = sub(xr[j], sh);
        if (out) orow[j] = xs;
        if (K > 0) softmax_digits(planes, ints, flag, xs, bs, K, (size_t)row * cols + j);
    }
}
// table[x] = floor(exp(log_theta - step * x) + 0.5)  (zksoftmax.cu:4-14); step = B_k / (sf_in sqrt d)
__global__ void __launch_bounds__(TPB) k_softmax_table(Fr* __restrict__ table, double log_theta, double step, uint32_t len) {
    const uint32_t x = blockIdx.x * TPB + threadIdx.x;
    if (x >= len) return;
    const double v = zkd::exp_det(log_theta - step * (double)x) + 0.5;
    table[x] = fr_from_u64((uint64_t)v);
}
// digits of -x in the mixed radix bs[0..K): plane k holds digit k (zksoftmax.cu:95-109).  Values whose
// negation does not fit 64 bits raise the flag (the reference leaves their planes unwritten).
__global__ void __launch_bounds__(TPB) k_softmax_decompose(const PlanePtrs planes, const IntPlanePtrs ints, uint32_t* __restrict__ flag, const Fr* __restrict__ X, const U32Pack8 bs,
                                                           int K, size_t n) {
    const size_t g = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (g < n) softmax_digits(planes, ints, flag, X[g], bs, K, g);
}

// ---- host side ----------------------------------------------------------------------------------------------------------------------
#define LAUNCH1D(kernel, n, st, ...)                                                         \
    do {                                                                                     \
        if ((n) > 0) {                                                                       \
            hipLaunchKernelGGL(kernel, dim3(cdiv((n), TPB)), dim3(TPB), 0, (hipStream_t)(st), __VA_ARGS__); \
            ZK_LAUNCH_CHECK();                                                               \
        }                                                                                    \
    } while (0)

static int read_flag(uint32_t* dev_flag, uint32_t* host_val, hipStream_t st) {
    void* stage = nullptr;
    int rc = staging(&stage, 4);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, dev_flag, 4, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    *host_val = *(uint32_t*)stage;
    return 0;
}

// eq table of k challenges into out (2^k elements, Montgomery form), queued on the stream; the two half tables live in the arena
static int eq_table_queue(Fr* out, const uint32_t* u, int k, Arena& arena, hipStream_t st) {
    EqChallenges c;
    Fr one = big_zero<8>();
    one.v[0] = 1;
    for (int j = 0; j < 30; ++j) {
        const Fr uj = j < k ? load_fr(u + 8 * j) : big_zero<8>();
        c.u[j] = to_mont(uj);
        c.omu[j] = to_mont(sub(one, uj));
    }
    const int kl = (k + 1) / 2, kh = k - kl;
    Scratch& half = arena.add(sizeof(Fr) * (((size_t)1 << kl) + ((size_t)1 << kh)));
    if (half.rc) return half.rc;
    Fr* lo = half.as<Fr>();
    Fr* hi = lo + ((size_t)1 << kl);
    const size_t n = (size_t)1 << k;
    hipLaunchKernelGGL(k_eq_halves, dim3(cdiv(((size_t)1 << kl) + ((size_t)1 << kh), TPB)), dim3(TPB), 0, st, lo, hi, c, kl, kh);
    hipLaunchKernelGGL(k_eq_outer, dim3(cdiv(n, TPB)), dim3(TPB), 0, st, out, lo, hi, kl, n);
    ZK_LAUNCH_CHECK();
    return 0;
}

// The split evaluation (k_me_split) from this many challenges on; ZKLLM_ME_SPLIT=0 keeps every evaluation on the pass over
// the full eq table (to compare: the results are the same).
static constexpr int ME_SPLIT_MIN_K = 16;
static bool me_split_on() { static const bool on = [] { const char* e = getenv("ZKLLM_ME_SPLIT"); return !(e && e[0] == '0'); }(); return on; }

// ---- folds of a tensor of 32-bit integers by eq weights ------------------------------------------------------------------
// A tensor whose elements are 32-bit signed integers (a weight: fixed-point values) folds from its int32 form: an eighth of
// the bytes, and a product with an eq entry is eight limb products with no reduction.  The unreduced sum of a whole fold
// fits ten limbs (entries below 2^255, magnitudes up to 2^31, up to 2^24 terms) and is reduced once: the low 256 bits by
// one Montgomery product with 1 (the entries carry R), the two limbs above them count R each, which that product cancels.
// id: unique per handle (the int32 form never changes once written).  src_*: set by zk_fr_gather_by_queries_ints -- element i
// is entry (queries[i] - src_low) of the table with that id, for every query inside the table.
struct FoldPrepared { int32_t* ints = nullptr; size_t n = 0; uint64_t id = 0, src_queries = 0, src_table = 0; int32_t src_low = 0; };
static uint64_t fold_prepared_id() { static std::mutex mu; static uint64_t next = 0; std::lock_guard<std::mutex> lk(mu); return ++next; }
struct EqPair { Fr e, ne; };        // an eq entry and its negative, Montgomery form
__global__ void __launch_bounds__(TPB) k_fold_ints(int32_t* __restrict__ out, uint32_t* __restrict__ bad, const Fr* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const Fr x = in[i];
    const int32_t v = fr_to_i32(x);
    out[i] = v;
    if (!equal(fr_from_i64((int64_t)v), x)) atomicOr(bad, 1u);
}
__global__ void __launch_bounds__(TPB) k_eq_pairs(EqPair* __restrict__ out, const Fr* __restrict__ E, uint32_t cur) {
    const uint32_t j = blockIdx.x * TPB + threadIdx.x;
    if (j >= cur) return;
    EqPair p;
    p.e = E[j];
    p.ne = neg(p.e);
    out[j] = p;
}
__device__ __forceinline__ void ifold_mac(uint32_t (&acc)[10], const Fr& e, const Fr& ne, int32_t w) {
    const bool ng = w < 0;
    const uint32_t a = ng ? 0u - (uint32_t)w : (uint32_t)w;
    uint64_t carry = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t s = ng ? ne.v[i] : e.v[i];
        const uint64_t t = (uint64_t)s * a + acc[i] + carry;       // at most (2^32 - 1)^2 + 2 (2^32 - 1) = 2^64 - 1
        acc[i] = (uint32_t)t;
        carry = t >> 32;
    }
    const uint64_t t = (uint64_t)acc[8] + carry;
    acc[8] = (uint32_t)t;
    acc[9] += (uint32_t)(t >> 32);
}
__device__ __forceinline__ Fr ifold_finish(const uint32_t (&acc)[10]) {
    Fr lo;
#pragma unroll
    for (int i = 0; i < 8; ++i) lo.v[i] = acc[i];
    lo = reduce_once(reduce_once(lo));          // below 2^256 < 3 r
    Fr one = big_zero<8>(), hi = big_zero<8>();
    one.v[0] = 1;
    hi.v[0] = acc[8];
    hi.v[1] = acc[9];
    return add(mont_mul(lo, one), hi);
}
// the unreduced sums of four waves through LDS: wave 0 adds them up
__device__ __forceinline__ void ifold_put(uint32_t (*sh)[10][64], uint32_t wv, uint32_t lane, const uint32_t (&acc)[10]) {
#pragma unroll
    for (int i = 0; i < 10; ++i) sh[wv][i][lane] = acc[i];
}
__device__ __forceinline__ void ifold_gather(uint32_t (&acc)[10], uint32_t (*sh)[10][64], uint32_t lane) {
#pragma unroll
    for (int q = 1; q < 4; ++q) {
        uint32_t c = 0;
#pragma unroll
        for (int i = 0; i < 10; ++i) acc[i] = addc32(acc[i], sh[q][i][lane], c);
    }
}
// out[o][w] = sum_j E[j] in[o][j][w].  A workgroup serves 64 consecutive outputs; each of its four waves takes a quarter of
// the axis (the entries of a step are the same for every lane of a wave), eight loads in flight per lane.
__global__ void __launch_bounds__(256) k_ifold_window(Fr* __restrict__ out, const int32_t* __restrict__ in, const EqPair* __restrict__ E, size_t n_out, uint32_t cur, size_t window) {
    __shared__ uint32_t sh[4][10][64];
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    const size_t g = (size_t)blockIdx.x * 64 + lane;
    const bool live = g < n_out;
    const size_t gg = live ? g : n_out - 1;
    const size_t o = gg / window, w = gg % window;
    const int32_t* p = in + o * (size_t)cur * window + w;
    const uint32_t per = (cur + 3) / 4;
    const uint32_t j0 = wv * per < cur ? wv * per : cur, j1 = j0 + per < cur ? j0 + per : cur;
    uint32_t acc[10];
#pragma unroll
    for (int i = 0; i < 10; ++i) acc[i] = 0;
    uint32_t j = j0;
    for (; j + 8 <= j1; j += 8) {
        int32_t x[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) x[t] = p[(size_t)(j + t) * window];
#pragma unroll
        for (int t = 0; t < 8; ++t) ifold_mac(acc, E[j + t].e, E[j + t].ne, x[t]);
    }
    for (; j < j1; ++j) ifold_mac(acc, E[j].e, E[j].ne, p[(size_t)j * window]);
    if (wv) ifold_put(sh, wv, lane, acc);
    __syncthreads();
    if (wv == 0) {
        ifold_gather(acc, sh, lane);
        if (live) out[g] = ifold_finish(acc);
    }
}
// the same fold of the elementwise product of two tensors in int32 form (exact 64-bit integers: sixteen limb products into a
// twelve-limb sum per element): the product is never written
__global__ void __launch_bounds__(256) k_ifold_window_prod(Fr* __restrict__ out, const int32_t* __restrict__ ina, const int32_t* __restrict__ inb, const EqPair* __restrict__ E,
                                                           size_t n_out, uint32_t cur, size_t window) {
    __shared__ uint32_t sh[4][12][64];
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    const size_t g = (size_t)blockIdx.x * 64 + lane;
    const bool live = g < n_out;
    const size_t gg = live ? g : n_out - 1;
    const size_t o = gg / window, w = gg % window;
    const size_t base = o * (size_t)cur * window + w;
    const uint32_t per = (cur + 3) / 4;
    const uint32_t j0 = wv * per < cur ? wv * per : cur, j1 = j0 + per < cur ? j0 + per : cur;
    uint32_t acc[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) acc[i] = 0;
    uint32_t j = j0;
    for (; j + 4 <= j1; j += 4) {
        int32_t x[4], y[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) { x[t] = ina[base + (size_t)(j + t) * window]; y[t] = inb[base + (size_t)(j + t) * window]; }
#pragma unroll
        for (int t = 0; t < 4; ++t) imac64(acc, E[j + t].e, E[j + t].ne, (int64_t)x[t], (int64_t)y[t]);
    }
    for (; j < j1; ++j) imac64(acc, E[j].e, E[j].ne, (int64_t)ina[base + (size_t)j * window], (int64_t)inb[base + (size_t)j * window]);
    if (wv) {
#pragma unroll
        for (int i = 0; i < 12; ++i) sh[wv][i][lane] = acc[i];
    }
    __syncthreads();
    if (wv == 0) {
#pragma unroll
        for (int q = 1; q < 4; ++q) {
            uint32_t c = 0;
#pragma unroll
            for (int i = 0; i < 12; ++i) acc[i] = addc32(acc[i], sh[q][i][lane], c);
        }
        if (live) out[g] = imac64_finish(acc);
    }
}
// window 1: out[o] = sum_j E[j] in[o][j].  A workgroup serves four rows; each of its four waves takes a quarter of the axis
// for all four (an entry is loaded once for the four rows), lanes over j, a butterfly over the wave, then the four waves' sums.
__global__ void __launch_bounds__(256) k_ifold_rows(Fr* __restrict__ out, const int32_t* __restrict__ in, const EqPair* __restrict__ E, size_t other, uint32_t cur) {
    __shared__ uint32_t sh[4][10][64];          // [wave][limb][row] (rows 0..3 used)
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    const size_t o0 = (size_t)blockIdx.x * 4;
    const uint32_t per = ((cur + 255) / 256) * 64;          // a quarter of the axis, in whole wave steps
    const uint32_t j0 = wv * per < cur ? wv * per : cur, j1 = j0 + per < cur ? j0 + per : cur;
    uint32_t acc[4][10];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 10; ++i) acc[r][i] = 0;
    for (uint32_t j = j0 + lane; j < j1; j += 64) {
        const EqPair ep = E[j];
        int32_t x[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) x[r] = o0 + r < other ? in[(o0 + r) * (size_t)cur + j] : 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) ifold_mac(acc[r], ep.e, ep.ne, x[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        for (int off = 32; off > 0; off >>= 1) {
            uint32_t c = 0;
#pragma unroll
            for (int i = 0; i < 10; ++i) acc[r][i] = addc32(acc[r][i], (uint32_t)__shfl_xor((int)acc[r][i], off, 64), c);
        }
        if (lane == 0 && wv) {
#pragma unroll
            for (int i = 0; i < 10; ++i) sh[wv][i][r] = acc[r][i];
        }
    }
    __syncthreads();
    if (wv == 0 && lane == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            ifold_gather(acc[r], sh, (uint32_t)r);
            if (o0 + r < other) out[o0 + r] = ifold_finish(acc[r]);
        }
    }
}

// out[i] = table[idx[i]] with the int32 form of the same elements beside it, both from the table's own int32 form
__global__ void __launch_bounds__(TPB) k_gather_ints(Fr* __restrict__ out, int32_t* __restrict__ out_ints, const Fr* __restrict__ /*table*/, const int32_t* __restrict__ table_ints,
                                                     const uint32_t* __restrict__ idx, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int32_t v = table_ints[idx[i]];      // the table's int32 form is an eighth of the table: it stays cached where the table does not
    out[i] = fr_from_i64((int64_t)v);           // the same element as table[idx[i]]
    out_ints[i] = v;
}
// out[i] = a[i] * b[i] for two tensors given by their int32 forms: the product is an exact 64-bit integer
__global__ void __launch_bounds__(TPB) k_mul_ints(Fr* __restrict__ out, const int32_t* __restrict__ a, const int32_t* __restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_from_i64((int64_t)a[i] * (int64_t)b[i]);
}
// out[i] = table[queries[i] - low] from the int32 forms of queries and table (a query outside the table reads entry 0: the index
// pass, run before, reports those)
__global__ void __launch_bounds__(TPB) k_gather_by_queries(Fr* __restrict__ out, int32_t* __restrict__ out_ints, const int32_t* __restrict__ queries, int32_t low,
                                                           const int32_t* __restrict__ table_ints, uint32_t N, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int64_t d = (int64_t)queries[i] - (int64_t)low;
    const uint32_t j = (d >= 0 && d < (int64_t)N) ? (uint32_t)d : 0u;
    const int32_t v = table_ints[j];
    if (out) out[i] = fr_from_i64((int64_t)v);
    out_ints[i] = v;
}
// Multilinear evaluations at one point of KF (0 or 1) tensors of field elements and KI tensors given in int32 form, in one
// pass over the point's eq table: an int32 element costs eight limb products into the lane's unreduced sum.
struct MeIntPtrs { const int32_t* x[6]; };
template <int KF, int KI> __global__ void __launch_bounds__(TPB) k_me_mixed(Fr* __restrict__ partials, const Fr* __restrict__ XF, const Fr* __restrict__ XF2, const MeIntPtrs pi,
                                                                            const Fr* __restrict__ E, size_t n) {
    Fr accf = big_zero<8>(), accf2 = big_zero<8>();
    uint32_t acc[KI][10];
#pragma unroll
    for (int k = 0; k < KI; ++k)
#pragma unroll
        for (int i = 0; i < 10; ++i) acc[k][i] = 0;
    const size_t stride = (size_t)gridDim.x * TPB;          // at most 2^27 / stride terms per lane: far below the 2^24 that fit
    for (size_t t = (size_t)blockIdx.x * TPB + threadIdx.x; t < n; t += stride) {
        const Fr e = E[t];
        const Fr ne = neg(e);
        int32_t x[KI];
#pragma unroll
        for (int k = 0; k < KI; ++k) x[k] = pi.x[k][t];
        if constexpr (KF >= 1) accf = add(accf, mont_mul(e, XF[t]));
        if constexpr (KF == 2) accf2 = add(accf2, mont_mul(e, XF2[t]));
#pragma unroll
        for (int k = 0; k < KI; ++k) ifold_mac(acc[k], e, ne, x[k]);
    }
    Fr out[KF + KI];
    if constexpr (KF >= 1) out[0] = accf;
    if constexpr (KF == 2) out[1] = accf2;
#pragma unroll
    for (int k = 0; k < KI; ++k) out[KF + k] = ifold_finish(acc[k]);
    block_reduce_store<KF + KI>(out, partials);
}

// ---- multilinear evaluations without the point's full eq table --------------------------------------------------------------
// eq(u, t) = lo[t mod 2^kl] * hi[t div 2^kl], so  sum_t X[t] eq(u, t) = sum_g lo[g] (sum_h X[h 2^kl + g] hi[h]).  A lane owns one
// g (and one slice of the h range): every step it multiplies its element by hi[h], the SAME value for all lanes of the wave,
// and adds the product to an unreduced sum -- an int32 element by eight limb products (ifold_mac), a field element by 81
// limb products on 29-bit limbs (wide29_mac; a carry pass every fourth term) -- and it reduces and multiplies by lo[g] once, at
// the end.  Against a pass over the full table (k_eq_outer writes it with one field product per entry, k_me_mixed reads it
// and pays a second one per field element) a field element costs about a sixth of the instructions, an int32 element a
// tenth, and the table's 64 bytes of traffic per position are gone.
// Tables: lo and hi as k_eq_halves leaves them (Montgomery form), the negatives of hi, and both with the factor 2^261 on
// 29-bit limbs (x 2^261 = 32 x R): the sum's reduction and the product with lo each take one 2^-261.
struct MeSplitTabs { const Fr* lo_m; const Fr* hi_m; const Fr* hi_neg; const Fr29* lo29; const Fr29* hi29; int kl; uint32_t nhi, per_slice; };
__global__ void __launch_bounds__(TPB) k_me_split_tabs(Fr* __restrict__ hi_neg, Fr29* __restrict__ lo29, Fr29* __restrict__ hi29, const Fr* __restrict__ lo_m,
                                                       const Fr* __restrict__ hi_m, uint32_t nlo, uint32_t nhi) {
    const uint32_t g = blockIdx.x * TPB + threadIdx.x;
    if (g >= nlo + nhi) return;
    Fr c32 = big_zero<8>();
    c32.v[0] = 32;
    c32 = to_mont(c32);
    if (g < nlo) lo29[g] = fr29_repack(mont_mul(lo_m[g], c32));
    else {
        const Fr h = hi_m[g - nlo];
        hi_neg[g - nlo] = neg(h);
        hi29[g - nlo] = fr29_repack(mont_mul(h, c32));
    }
}
template <int KF, int KI> __global__ void __launch_bounds__(TPB) k_me_split(Fr* __restrict__ partials, const Fr* __restrict__ XF, const Fr* __restrict__ XF2, const MeIntPtrs pi,
                                                                            const MeSplitTabs tb, size_t n) {
    const uint32_t gid = blockIdx.x * TPB + threadIdx.x;
    const uint32_t g = gid & ((1u << tb.kl) - 1u), slice = gid >> tb.kl;
    const uint32_t h0 = slice * tb.per_slice, h1 = h0 + tb.per_slice < tb.nhi ? h0 + tb.per_slice : tb.nhi;
    Wide29 w[KF > 0 ? KF : 1];
    uint32_t acc[KI > 0 ? KI : 1][10];
#pragma unroll
    for (int k = 0; k < KF; ++k) w[k] = wide29_zero();
#pragma unroll
    for (int k = 0; k < KI; ++k)
#pragma unroll
        for (int i = 0; i < 10; ++i) acc[k][i] = 0;
    for (uint32_t h = h0; h < h1; ++h) {
        const size_t t = ((size_t)h << tb.kl) + g;
        if (t < n) {
            if constexpr (KI > 0) {
                const Fr e = tb.hi_m[h], ne = tb.hi_neg[h];
                int32_t x[KI];
#pragma unroll
                for (int k = 0; k < KI; ++k) x[k] = pi.x[k][t];
#pragma unroll
                for (int k = 0; k < KI; ++k) ifold_mac(acc[k], e, ne, x[k]);
            }
            if constexpr (KF > 0) {
                const Fr29 e29 = tb.hi29[h];
                wide29_mac(w[0], fr29_repack(XF[t]), e29);
                if constexpr (KF == 2) wide29_mac(w[1], fr29_repack(XF2[t]), e29);
            }
        }
        if constexpr (KF > 0) {
            if (((h - h0) & 3u) == 3u) {
#pragma unroll
                for (int k = 0; k < KF; ++k) wide29_carry(w[k]);
            }
        }
    }
    Fr out[KF + KI];
    if constexpr (KF > 0) {
        const Fr29 l29 = tb.lo29[g];
#pragma unroll
        for (int k = 0; k < KF; ++k) out[k] = fr29_canon_pack(fr29_mul(wide29_redc(w[k]), l29));
    }
    if constexpr (KI > 0) {
        const Fr l = tb.lo_m[g];
#pragma unroll
        for (int k = 0; k < KI; ++k) out[KF + k] = mont_mul(ifold_finish(acc[k]), l);
    }
    block_reduce_store<KF + KI>(out, partials);
}
// the tables of k_me_split for k challenges and n elements, queued on the stream (they live in the arena); blocks: its grid
static int me_split_tabs_queue(MeSplitTabs& tb, unsigned& blocks, const uint32_t* u, int k, size_t n, Arena& arena, hipStream_t st) {
    EqChallenges c;
    Fr one = big_zero<8>();
    one.v[0] = 1;
    for (int j = 0; j < 30; ++j) {
        const Fr uj = j < k ? load_fr(u + 8 * j) : big_zero<8>();
        c.u[j] = to_mont(uj);
        c.omu[j] = to_mont(sub(one, uj));
    }
    const int kl = (k + 1) / 2, kh = k - kl;
    const uint32_t nlo = 1u << kl, nhi_full = 1u << kh;
    Scratch& half = arena.add(sizeof(Fr) * ((size_t)nlo + 2 * (size_t)nhi_full));
    Scratch& t29 = arena.add(sizeof(Fr29) * ((size_t)nlo + nhi_full));
    if (half.rc) return half.rc;
    if (t29.rc) return t29.rc;
    Fr* lo = half.as<Fr>();
    Fr* hi = lo + nlo;
    Fr* hi_neg = hi + nhi_full;
    Fr29* lo29 = t29.as<Fr29>();
    Fr29* hi29 = lo29 + nlo;
    hipLaunchKernelGGL(k_eq_halves, dim3(cdiv((size_t)nlo + nhi_full, TPB)), dim3(TPB), 0, st, lo, hi, c, kl, kh);
    hipLaunchKernelGGL(k_me_split_tabs, dim3(cdiv((size_t)nlo + nhi_full, TPB)), dim3(TPB), 0, st, hi_neg, lo29, hi29, lo, hi, nlo, nhi_full);
    ZK_LAUNCH_CHECK();
    const uint32_t nhi = (uint32_t)((n + nlo - 1) / nlo);          // rows that hold elements
    // slices of the h range: at most 1024 terms in a lane's unreduced sums, and 2^17 lanes where the tensor is large enough
    uint32_t S = 1;
    while ((nhi + S - 1) / S > 1024 || ((size_t)nlo * S < ((size_t)1 << 17) && S < nhi)) S <<= 1;
    tb.lo_m = lo; tb.hi_m = hi; tb.hi_neg = hi_neg; tb.lo29 = lo29; tb.hi29 = hi29;
    tb.kl = kl; tb.nhi = nhi; tb.per_slice = (nhi + S - 1) / S;
    blocks = (unsigned)(((size_t)nlo * S) / TPB);
    return 0;
}


extern "C" {

int zk_lookup_index_fr(void* idx_u32, const void* vals, int32_t low, uint32_t table_size, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (n == 0) return 0;
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    LAUNCH1D(k_index_fr, n, st, (uint32_t*)idx_u32, flag.as<uint32_t>(), (const Fr*)vals, fr_from_i64((int64_t)low), table_size, n);
    uint32_t f = 0;
    int rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    ZK_ARG(f == 0, "lookup: a value lies outside the table range");
    return 0;
}
int zk_lookup_index_i32(void* idx_u32, const void* vals_i32, int32_t low, uint32_t table_size, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (n == 0) return 0;
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    LAUNCH1D(k_index_i32, n, st, (uint32_t*)idx_u32, flag.as<uint32_t>(), (const int32_t*)vals_i32, low, table_size, n);
    uint32_t f = 0;
    int rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    ZK_ARG(f == 0, "lookup: a value lies outside the table range");
    return 0;
}
// counts[0..nbins) = number of occurrences of each index (zeroed here first)
static int hist_queue(uint32_t* counts, const KeySrc src, size_t n, uint32_t nbins, hipStream_t st) {
    ZK_HIP(hipMemsetAsync(counts, 0, sizeof(uint32_t) * (size_t)nbins, st));
    if (n == 0) return 0;
    if (nbins <= HIST_LDS_BINS) {
        unsigned blocks = cdiv(n, (size_t)TPB * 16);
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(k_hist_lds, dim3(blocks), dim3(TPB), 0, st, counts, src, n, nbins);
    } else if (n >= HP_MIN_QUERIES && n < ((size_t)1 << 32) && nbins <= HP_MAXP * HP_BINS) {
        return hist_partitioned(counts, src, n, nbins, st);
    } else {
        hipLaunchKernelGGL(k_hist_global, dim3(cdiv(n, (size_t)TPB * HH_PER_LANE)), dim3(TPB), 0, st, counts, src, n);
    }
    ZK_LAUNCH_CHECK();
    return 0;
}
int zk_lookup_hist(void* counts_u32, const void* idx_u32, size_t n, uint32_t nbins, void* stv) {
    ZK_ARG(nbins >= 1, "zk_lookup_hist: no bins");
    return hist_queue((uint32_t*)counts_u32, KeySrc{(const uint32_t*)idx_u32, nullptr, 0, 0, nullptr}, n, nbins, (hipStream_t)stv);
}
// zk_lookup_index_i32 and zk_lookup_hist in one: the counting passes form the positions value - low themselves, no array of
// them is written.  A value outside [low, low + len) is an error, as there.
int zk_lookup_hist_i32(void* counts_u32, const void* vals_i32, int32_t low, uint32_t len, size_t n, uint32_t nbins, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(nbins >= 1 && len >= 1 && len <= nbins, "zk_lookup_hist_i32: need 1 <= len <= nbins");
    ZK_ARG(vals_i32 != nullptr || n == 0, "zk_lookup_hist_i32: null queries");
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    int rc = hist_queue((uint32_t*)counts_u32, KeySrc{nullptr, (const int32_t*)vals_i32, low, len, flag.as<uint32_t>()}, n, nbins, st);
    if (rc) return rc;
    uint32_t f = 0;
    rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    ZK_ARG(f == 0, "lookup: a value lies outside the table range");
    return 0;
}
int zk_range_table(void* table, int32_t low, uint32_t len, uint32_t table_size, void* st) {
    ZK_ARG(len >= 1 && table_size >= len, "zk_range_table: need 1 <= len <= table_size");
    LAUNCH1D(k_range_table, table_size, st, (Fr*)table, low, len, table_size);
    return 0;
}
// out[i] = 1 / (in[i] + beta), standard form; 0 where in[i] + beta == 0 (tlookup_inv_kernel tlookup.cu:50-62)
int zk_fr_batch_inv(void* out, const void* in, const uint32_t* beta, size_t n, void* st) {
    if (n == 0) return 0;
    Arena tmp((hipStream_t)st);
    // large inputs use scratch memory that goes back to the allocator when this returns, remembered as last used on `st`
    return batch_inv_queue((Fr*)out, (const Fr*)in, load_fr(beta), n, tmp, (hipStream_t)st);
}
// E[t] for t < 2^k (Montgomery form) from k standard-form challenges; out holds 2^k elements
int zk_eq_table(void* out, const uint32_t* u, int k, void* stv) {
    ZK_ARG(k >= 0 && k <= 30, "zk_eq_table: k out of range");
    Arena tmp((hipStream_t)stv);        // the half tables return to the allocator at once: later users are ordered behind these launches on the same stream
    return eq_table_queue((Fr*)out, u, k, tmp, (hipStream_t)stv);
}
// ---- folds of a tensor of 32-bit integers by eq weights ------------------------------------------------------------------
int zk_fr_fold_prepare(void** prepared, const void* t, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(prepared != nullptr && t != nullptr && n >= 1, "zk_fr_fold_prepare: null argument or empty tensor");
    *prepared = nullptr;
    void* ints = nullptr;
    int rc = pool_alloc(&ints, sizeof(int32_t) * n, st);
    if (rc) return rc;
    uint32_t bad = 0;
    {
        Scratch flag(4, st);
        if (flag.rc) { pool_free(ints, st); return flag.rc; }
        hipError_t e = hipMemsetAsync(flag.p, 0, 4, st);        // setup call: never part of a captured graph (it ends with a host read)
        if (e != hipSuccess) { pool_free(ints, st); ZK_HIP(e); }
        hipLaunchKernelGGL(k_fold_ints, dim3(cdiv(n, TPB)), dim3(TPB), 0, st, (int32_t*)ints, flag.as<uint32_t>(), (const Fr*)t, n);
        rc = read_flag(flag.as<uint32_t>(), &bad, st);
    }
    if (rc || bad) { pool_free(ints, st); return rc; }
    FoldPrepared* fp = new FoldPrepared;
    fp->ints = (int32_t*)ints;
    fp->n = n;
    fp->id = fold_prepared_id();
    *prepared = fp;
    return 0;
}
int zk_fr_fold_prepared_free(void* prepared) {
    FoldPrepared* fp = (FoldPrepared*)prepared;
    if (!fp) return 0;
    pool_free(fp->ints, nullptr);
    delete fp;
    return 0;
}
int zk_fr_fold_prepared_new(void** prepared, void** ints_dev, size_t n, void* stv) {
    ZK_ARG(prepared != nullptr && ints_dev != nullptr && n >= 1, "zk_fr_fold_prepared_new: null argument or empty tensor");
    *prepared = nullptr;
    void* ints = nullptr;
    int rc = pool_alloc(&ints, sizeof(int32_t) * n, (hipStream_t)stv);
    if (rc) return rc;
    FoldPrepared* fp = new FoldPrepared;
    fp->ints = (int32_t*)ints;
    fp->n = n;
    fp->id = fold_prepared_id();
    *prepared = fp;
    *ints_dev = ints;
    return 0;
}
const void* zk_fr_fold_prepared_ints(const void* prepared) { return prepared ? ((const FoldPrepared*)prepared)->ints : nullptr; }
// The int32 form of a handle was written again (by anything but the kernel queued right after zk_fr_fold_prepared_new): the
// handle becomes a new form -- a fresh id, so that whatever remembered the old one (the outputs gathered by these queries or from
// this table) no longer counts as gathered from it, and nothing it was itself gathered from.
int zk_fr_fold_prepared_touch(void* prepared) {
    FoldPrepared* fp = (FoldPrepared*)prepared;
    ZK_ARG(fp != nullptr, "zk_fr_fold_prepared_touch: null handle");
    fp->id = fold_prepared_id();
    fp->src_queries = fp->src_table = 0;
    fp->src_low = 0;
    return 0;
}
int zk_fr_gather_ints(void* out, void* out_ints, const void* table, const void* table_prepared, const void* idx, size_t n, void* stv) {
    const FoldPrepared* tp = (const FoldPrepared*)table_prepared;
    ZK_ARG(out != nullptr && out_ints != nullptr && table != nullptr && tp != nullptr && idx != nullptr, "zk_fr_gather_ints: null argument");
    LAUNCH1D(k_gather_ints, n, stv, (Fr*)out, (int32_t*)out_ints, (const Fr*)table, tp->ints, (const uint32_t*)idx, n);
    return 0;
}
int zk_fr_gather_by_queries_ints(void* out, void* out_prepared, const void* queries_prepared, int32_t low, const void* table_prepared, size_t n, void* stv) {
    FoldPrepared* o = (FoldPrepared*)out_prepared;
    const FoldPrepared *q = (const FoldPrepared*)queries_prepared, *t = (const FoldPrepared*)table_prepared;
    ZK_ARG(o != nullptr && q != nullptr && t != nullptr, "zk_fr_gather_by_queries_ints: null argument");      // out may be null: only the int32 form is written
    ZK_ARG(o->n == n && q->n == n && t->n >= 1 && t->n <= 0xFFFFFFFFu, "zk_fr_gather_by_queries_ints: int32 forms of another size");
    LAUNCH1D(k_gather_by_queries, n, stv, (Fr*)out, o->ints, q->ints, low, t->ints, (uint32_t)t->n, n);
    o->src_queries = q->id;
    o->src_table = t->id;
    o->src_low = low;
    return 0;
}
int zk_fr_mul_ints(void* out, const void* a_prepared, const void* b_prepared, size_t n, void* stv) {
    const FoldPrepared *a = (const FoldPrepared*)a_prepared, *b = (const FoldPrepared*)b_prepared;
    ZK_ARG(out != nullptr && a != nullptr && b != nullptr && a->n == n && b->n == n, "zk_fr_mul_ints: null argument or int32 forms of another size");
    LAUNCH1D(k_mul_ints, n, stv, (Fr*)out, a->ints, b->ints, n);
    return 0;
}
int zk_fr_me_multi_ints(uint32_t* out_host, const void* const* Xs, const void* const* prepareds, int K, size_t n, const uint32_t* u, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(K >= 1 && K <= 8, "zk_fr_me_multi_ints: 1..8 tensors");
    ZK_ARG(k >= 0 && k <= 30 && n >= 1 && n <= ((size_t)1 << k) && (k == 0 || n > ((size_t)1 << (k - 1))), "zk_fr_me_multi_ints: n does not match the number of challenges");
    // Every tensor with an int32 form is read from that form and never as field elements (a tensor that keeps only its int32
    // form may have nothing written there): they go through the mixed kernel six at a time, with up to two tensors of field
    // elements riding along on the first pass; what is left of those is evaluated as zk_fr_me_multi does.
    int ints_at[8], n_ints = 0, fr_at[8], n_fr = 0;
    for (int i = 0; i < K; ++i) {
        const FoldPrepared* fp = prepareds ? (const FoldPrepared*)prepareds[i] : nullptr;
        ZK_ARG(!fp || fp->n == n, "zk_fr_me_multi_ints: an int32 form of another size");
        if (fp) ints_at[n_ints++] = i;
        else fr_at[n_fr++] = i;
    }
    if (n_ints == 0) return zk_fr_me_multi(out_host, Xs, K, n, u, k, stv);
    Arena tmp(st);
    const bool split = me_split_on() && k >= ME_SPLIT_MIN_K;
    MeSplitTabs tb;
    unsigned nb = reduce_grid(n);
    Fr* Eptr = nullptr;
    int rc = 0;
    if (split) rc = me_split_tabs_queue(tb, nb, u, k, n, tmp, st);
    else {
        Scratch& E = tmp.add(sizeof(Fr) * ((size_t)1 << k));
        if (E.rc) return E.rc;
        rc = eq_table_queue(E.as<Fr>(), u, k, tmp, st);
        Eptr = E.as<Fr>();
    }
    if (rc) return rc;
    Scratch& part = tmp.add(sizeof(Fr) * 8 * nb);
    if (part.rc) return part.rc;
    int fr_done = 0;
    for (int i0 = 0; i0 < n_ints; i0 += 6) {
        const int ni = n_ints - i0 < 6 ? n_ints - i0 : 6;
        const int KF = i0 == 0 ? (n_fr >= 2 && ni <= 3 ? 2 : (n_fr ? 1 : 0)) : 0, KT = KF + ni;         // two tensors of field elements ride along with up to three int32 forms
        MeIntPtrs pi;
        for (int i = 0; i < 6; ++i) pi.x[i] = ((const FoldPrepared*)prepareds[ints_at[i0 + (i < ni ? i : 0)]])->ints;
        const Fr* XF = KF ? (const Fr*)Xs[fr_at[0]] : nullptr;
        const Fr* XF2 = KF == 2 ? (const Fr*)Xs[fr_at[1]] : nullptr;
#define MEI_CASE(F, I)                                                                                                                      \
    if (KF == F && ni == I) {                                                                                                               \
        if (split) hipLaunchKernelGGL((k_me_split<F, I>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), XF, XF2, pi, tb, n);                 \
        else hipLaunchKernelGGL((k_me_mixed<F, I>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), XF, XF2, pi, Eptr, n);                      \
    }
        MEI_CASE(0, 1) MEI_CASE(0, 2) MEI_CASE(0, 3) MEI_CASE(0, 4) MEI_CASE(0, 5) MEI_CASE(0, 6)
        MEI_CASE(1, 1) MEI_CASE(1, 2) MEI_CASE(1, 3) MEI_CASE(1, 4) MEI_CASE(1, 5) MEI_CASE(1, 6)
        MEI_CASE(2, 1) MEI_CASE(2, 2) MEI_CASE(2, 3)
#undef MEI_CASE
        ZK_LAUNCH_CHECK();
        Fr s8[8];
        rc = finish_sums(part.as<Fr>(), nb, KT, 0, s8, st);
        if (rc) return rc;
        for (int i = 0; i < KF; ++i) memcpy(out_host + 8 * fr_at[i], &s8[i], sizeof(Fr));
        for (int i = 0; i < ni; ++i) memcpy(out_host + 8 * ints_at[i0 + i], &s8[KF + i], sizeof(Fr));
        fr_done += KF;
    }
    if (n_fr > fr_done) {         // the other tensors of field elements
        const void* rest[8];
        for (int i = fr_done; i < n_fr; ++i) rest[i - fr_done] = Xs[fr_at[i]];
        Fr r8[8];
        rc = zk_fr_me_multi((uint32_t*)r8, rest, n_fr - fr_done, n, u, k, stv);
        if (rc) return rc;
        for (int i = fr_done; i < n_fr; ++i) memcpy(out_host + 8 * fr_at[i], &r8[i - fr_done], sizeof(Fr));
    }
    return 0;
}
int zk_fr_fold_axis_prepared(void* out, const void* prepared, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    const FoldPrepared* fp = (const FoldPrepared*)prepared;
    ZK_ARG(fp != nullptr && out != nullptr && u != nullptr, "zk_fr_fold_axis_prepared: null argument");
    ZK_ARG(levels >= 1 && levels <= 24, "zk_fr_fold_axis_prepared: 1 to 24 levels");
    ZK_ARG(cur >= 1 && cur <= (1u << levels), "zk_fr_fold_axis_prepared: the axis is longer than 2^levels");
    ZK_ARG(other >= 1 && window >= 1 && other * (size_t)cur * window == fp->n, "zk_fr_fold_axis_prepared: other * cur * window is not the tensor's size");
    Arena tmp(st);
    Scratch& E = tmp.add(sizeof(Fr) * ((size_t)1 << levels));
    Scratch& P = tmp.add(sizeof(EqPair) * (size_t)cur);
    if (E.rc) return E.rc;
    if (P.rc) return P.rc;
    int rc = eq_table_queue(E.as<Fr>(), u, levels, tmp, st);
    if (rc) return rc;
    hipLaunchKernelGGL(k_eq_pairs, dim3(cdiv(cur, TPB)), dim3(TPB), 0, st, P.as<EqPair>(), E.as<Fr>(), cur);
    const size_t n_out = other * window;
    if (window == 1 && cur >= 64) hipLaunchKernelGGL(k_ifold_rows, dim3(cdiv(other, 4)), dim3(256), 0, st, (Fr*)out, fp->ints, P.as<EqPair>(), other, cur);
    else hipLaunchKernelGGL(k_ifold_window, dim3(cdiv(n_out, 64)), dim3(256), 0, st, (Fr*)out, fp->ints, P.as<EqPair>(), n_out, cur, window);
    ZK_LAUNCH_CHECK();
    return 0;
}
// zk_fr_fold_axis_prepared for the elementwise product of two tensors given by their int32 forms (n = other * cur * window
// elements each): out[o][w] = sum_j eq(u, j) a[o][j][w] b[o][j][w]
int zk_fr_fold_axis_prod(void* out, const void* a_prepared, const void* b_prepared, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    const FoldPrepared *fa = (const FoldPrepared*)a_prepared, *fb = (const FoldPrepared*)b_prepared;
    ZK_ARG(fa != nullptr && fb != nullptr && out != nullptr && u != nullptr, "zk_fr_fold_axis_prod: null argument");
    ZK_ARG(levels >= 1 && levels <= 24, "zk_fr_fold_axis_prod: 1 to 24 levels");
    ZK_ARG(cur >= 1 && cur <= (1u << levels), "zk_fr_fold_axis_prod: the axis is longer than 2^levels");
    ZK_ARG(other >= 1 && window >= 1 && other * (size_t)cur * window == fa->n && fb->n == fa->n, "zk_fr_fold_axis_prod: other * cur * window is not the tensors' size");
    Arena tmp(st);
    Scratch& E = tmp.add(sizeof(Fr) * ((size_t)1 << levels));
    Scratch& P = tmp.add(sizeof(EqPair) * (size_t)cur);
    if (E.rc) return E.rc;
    if (P.rc) return P.rc;
    int rc = eq_table_queue(E.as<Fr>(), u, levels, tmp, st);
    if (rc) return rc;
    hipLaunchKernelGGL(k_eq_pairs, dim3(cdiv(cur, TPB)), dim3(TPB), 0, st, P.as<EqPair>(), E.as<Fr>(), cur);
    const size_t n_out = other * window;
    hipLaunchKernelGGL(k_ifold_window_prod, dim3(cdiv(n_out, 64)), dim3(256), 0, st, (Fr*)out, fa->ints, fb->ints, P.as<EqPair>(), n_out, cur, window);
    ZK_LAUNCH_CHECK();
    return 0;
}
// out_host[i] = multilinear extension of Xs[i] (n elements each, zero beyond) at u (k challenges, 2^(k-1) < n <= 2^k)
int zk_fr_me_multi(uint32_t* out_host, const void* const* Xs, int K, size_t n, const uint32_t* u, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(K >= 1 && K <= 8, "zk_fr_me_multi: 1..8 tensors");
    ZK_ARG(k >= 0 && k <= 30 && n >= 1 && n <= ((size_t)1 << k) && (k == 0 || n > ((size_t)1 << (k - 1))), "zk_fr_me_multi: n does not match the number of challenges");
    Arena tmp(st);
    if (me_split_on() && k >= ME_SPLIT_MIN_K) {          // two tensors a pass, no eq table of the whole point
        MeSplitTabs tb;
        unsigned nb = 0;
        int rc = me_split_tabs_queue(tb, nb, u, k, n, tmp, st);
        if (rc) return rc;
        Scratch& part = tmp.add(sizeof(Fr) * 2 * nb);
        if (part.rc) return part.rc;
        const MeIntPtrs none = {};
        for (int i = 0; i < K; i += 2) {
            const int kf = K - i >= 2 ? 2 : 1;
            if (kf == 2) hipLaunchKernelGGL((k_me_split<2, 0>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), (const Fr*)Xs[i], (const Fr*)Xs[i + 1], none, tb, n);
            else hipLaunchKernelGGL((k_me_split<1, 0>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), (const Fr*)Xs[i], (const Fr*)nullptr, none, tb, n);
            ZK_LAUNCH_CHECK();
            Fr s2[2];
            rc = finish_sums(part.as<Fr>(), nb, kf, 0, s2, st);
            if (rc) return rc;
            memcpy(out_host + 8 * i, s2, sizeof(Fr) * kf);
        }
        return 0;
    }
    Scratch& E = tmp.add(sizeof(Fr) * ((size_t)1 << k));
    if (E.rc) return E.rc;
    int rc = eq_table_queue(E.as<Fr>(), u, k, tmp, st);
    if (rc) return rc;
    const unsigned nb = reduce_grid(n);
    Scratch& part = tmp.add(sizeof(Fr) * K * nb);
    if (part.rc) return part.rc;
    MePtrs p;
    for (int i = 0; i < 8; ++i) p.x[i] = (const Fr*)Xs[i < K ? i : 0];
#define ME_CASE(KK) case KK: hipLaunchKernelGGL(k_me_multi<KK>, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), p, E.as<Fr>(), n); break;
    switch (K) { ME_CASE(1) ME_CASE(2) ME_CASE(3) ME_CASE(4) ME_CASE(5) ME_CASE(6) ME_CASE(7) ME_CASE(8) }
#undef ME_CASE
    ZK_LAUNCH_CHECK();
    Fr s8[8];
    rc = finish_sums(part.as<Fr>(), nb, K, 0, s8, st);
    if (rc) return rc;
    memcpy(out_host, s8, sizeof(Fr) * K);
    return 0;
}
int zk_eq_halve(void* out, const void* in, size_t n_out, void* st) {
    LAUNCH1D(k_eq_halve, n_out, st, (Fr*)out, (const Fr*)in, n_out);
    return 0;
}
// One round of the lookup sumcheck over tensors of 2*n_out elements.  sums_host receives 5 values
// (phase 1) or 11 (phase 2), all in standard form; new_* receive the tensors folded by v.  B, T, m and
// their outputs are ignored in phase 1.
int zk_lookup_round(uint32_t* sums_host, void* nA, void* nS, void* nB, void* nT, void* nm, const void* A, const void* S, const void* B, const void* T,
                    const void* m, const void* E, const uint32_t* beta, const uint32_t* v, size_t n_out, int phase2, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(n_out >= 1, "zk_lookup_round: empty round");
    const unsigned nb = reduce_grid(n_out);
    const int K = phase2 ? 11 : 5;
    Scratch part(sizeof(Fr) * K * nb, st);
    if (part.rc) return part.rc;
    const Fr b = load_fr(beta), vm = to_mont(load_fr(v));
    if (phase2)
        hipLaunchKernelGGL(k_lookup_round<true>, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), (Fr*)nA, (Fr*)nS, (Fr*)nB, (Fr*)nT, (Fr*)nm, (const Fr*)A, (const Fr*)S,
                           (const Fr*)B, (const Fr*)T, (const Fr*)m, (const Fr*)E, b, vm, n_out, (Fr*)nullptr);
    else
        hipLaunchKernelGGL(k_lookup_round<false>, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), (Fr*)nA, (Fr*)nS, (Fr*)nullptr, (Fr*)nullptr, (Fr*)nullptr, (const Fr*)A,
                           (const Fr*)S, (const Fr*)nullptr, (const Fr*)nullptr, (const Fr*)nullptr, (const Fr*)E, b, vm, n_out, (Fr*)nullptr);
    ZK_LAUNCH_CHECK();
    Fr s[11];
    int rc = finish_sums(part.as<Fr>(), nb, K, 0, s, st);
    if (rc) return rc;
    // E carries R, each inner product one R^-1, the outer product with E another: sums 0..2, 5..7 and the
    // plain products 8..10 need one multiplication by R; sums 3, 4 are already standard.
    for (int i = 0; i < K; ++i)
        if (i != 3 && i != 4) s[i] = to_mont(s[i]);
    memcpy(sums_host, s, sizeof(Fr) * K);
    return 0;
}
// One round of multi_hadamard_sumchecks for K tensors of 2*n_out elements (K = 1..4).
// coefs_host: K+1 coefficients of sum_t E[t] prod_k (X0_k + x dX_k); new_Xs[k] receive the folds by v.
int zk_hadamard_round(uint32_t* coefs_host, void* const* new_Xs, const void* const* Xs, int K, const void* E, const uint32_t* v, size_t n_out, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(K >= 1 && K <= 4, "zk_hadamard_round: K must be 1..4");
    ZK_ARG(n_out >= 1, "zk_hadamard_round: empty round");
    const unsigned nb = reduce_grid(n_out);
    Scratch part(sizeof(Fr) * (K + 1) * nb, st);
    if (part.rc) return part.rc;
    const Fr vm = to_mont(load_fr(v));
#define HAD_CASE(KK)                                                                                                           \
    case KK: {                                                                                                                 \
        PtrPack<KK> p;                                                                                                         \
        for (int i = 0; i < KK; ++i) { p.in[i] = (const Fr*)Xs[i]; p.out[i] = (Fr*)new_Xs[i]; }                                 \
        hipLaunchKernelGGL(k_hadamard_round<KK>, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), p, (const Fr*)E, vm, n_out, (Fr*)nullptr); \
        break;                                                                                                                 \
    }
    switch (K) { HAD_CASE(1) HAD_CASE(2) HAD_CASE(3) HAD_CASE(4) }
#undef HAD_CASE
    ZK_LAUNCH_CHECK();
    Fr s[5];
    // e (= E*R) times a standard-form coefficient leaves no Montgomery factor: nothing to correct
    int rc = finish_sums(part.as<Fr>(), nb, K + 1, 0, s, st);
    if (rc) return rc;
    memcpy(coefs_host, s, sizeof(Fr) * (K + 1));
    return 0;
}
// ---- whole sumchecks as jobs ---------------------------------------------------------------------------------------------------
// A job queues every kernel of a sumcheck on one stream without a host round trip (the challenges are known up front),
// keeps its buffers until the results have been fetched, and can run on a stream of the library's own beside the caller.
// An eq table that several jobs read: the sumchecks of one softmax proof (its Hadamard argument and every segment's lookup)
// are all weighted by the same challenges, so the table -- 2 GB for the stacked attention -- is built by the first job that
// asks and the others wait for its event.  The jobs only read it (a round writes the next, shorter table elsewhere).
// Freed when the last holder lets go: every job holds it until its own completion has been seen on the host, and the slot
// below holds the latest one until another table replaces it.
struct SharedEq {
    void* p = nullptr;
    hipEvent_t ready = nullptr;
    int k = 0;
    std::vector<uint32_t> key;
    ~SharedEq() {
        if (ready) (void)hipEventDestroy(ready);
        if (p) (void)pool_free(p, nullptr, true);      // every reader has finished (see above)
    }
};
static std::mutex g_eq_mu;
static std::shared_ptr<SharedEq>& g_eq_latest = *new std::shared_ptr<SharedEq>();      // never destroyed: no device call after the runtime has gone
struct SumJob {
    std::shared_ptr<SharedEq> eq;
    Arena arena;
    hipStream_t st = nullptr;
    Fr* sums = nullptr;          // rounds x per_round values
    Fr* extra = nullptr;         // one more value fetched with the sums (lookup: <B, m> with R^-1 attached), or null
    int rounds = 0, per_round = 0, n1 = 0;
    hipEvent_t ready = nullptr;
    void* host = nullptr;        // jobs on a side stream: pinned buffer the results are copied to behind the last kernel ...
    hipEvent_t done = nullptr;   // ... and the event behind that copy
    const uint32_t* n_ok_dev = nullptr;      // lookup jobs over int32 forms: the consistent prefix of the table (HintSrc::n_ok) ...
    uint32_t n_table = 0;                    // ... and the table's size
    // a job whose launches were handed to the library's launch thread: the ticket to wait for before anything of the job is
    // read, and what that thread's attempt returned
    uint64_t ticket = 0;
    int queue_rc = 0;
    std::string queue_err;
    // A job whose weights are an eq table of the library's own: summing the top variable out of eq(u, .) leaves its lower half
    // divided by 1 - u_top, so every round's table is the first table's prefix times a constant and no round writes a table --
    // the rounds read the prefix, and the E-weighted sums of round r are multiplied by eq_scale[r] when they are collected
    // (Montgomery form; empty: the rounds write their tables).  tail_from: the round the last-rounds kernel starts at (it
    // folds its table itself, from the prefix: its rounds share that round's constant).
    std::vector<Fr> eq_scale;
    int tail_from = -1;
};
// eq_scale of a job over `rounds` rounds whose table is eq(u_eq, .) of rounds - 1 challenges (index bit j <-> u_eq[j]); false
// (and nothing written) if some challenge is 1
static bool eq_prefix_scales(std::vector<Fr>& out, const uint32_t* u_eq, int rounds) {
    const int k = rounds - 1;
    std::vector<Fr> c((size_t)rounds);
    const Fr one = big_one_mont<8>();
    if (rounds >= 1) c[0] = one;
    for (int r = 1; r < rounds; ++r) {
        const Fr d = sub(one, to_mont(load_fr(u_eq + 8 * (size_t)(k - r))));
        if (is_zero(d)) return false;
        c[r] = mont_mul(c[r - 1], mont_inverse(d));
    }
    out.swap(c);
    return true;
}
// the E-weighted entries of collected sums (bit i of `weighted`: entry i of a round's per_round) times their round's constant
static bool eq_prefix_on() { static const bool on = [] { const char* e = getenv("ZKLLM_EQ_PREFIX"); return !(e && e[0] == '0'); }(); return on; }
static void eq_prefix_apply(const SumJob& job, Fr* sums, uint32_t weighted) {
    if (job.eq_scale.empty()) return;
    for (int r = 0; r < job.rounds; ++r) {
        const Fr& c = job.eq_scale[(size_t)((job.tail_from >= 0 && r > job.tail_from) ? job.tail_from : r)];
        for (int i = 0; i < job.per_round; ++i)
            if ((weighted >> i) & 1u) sums[(size_t)r * job.per_round + i] = mont_mul(sums[(size_t)r * job.per_round + i], c);
    }
}
__global__ void __launch_bounds__(64) k_u32_set(uint32_t* __restrict__ p, uint32_t v) { if (threadIdx.x == 0) *p = v; }
__global__ void __launch_bounds__(TPB) k_dot_part(Fr* __restrict__ partials, const Fr* __restrict__ a, const Fr* __restrict__ b, size_t n) {
    Fr acc[1] = {big_zero<8>()};
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (size_t)gridDim.x * TPB) acc[0] = add(acc[0], mont_mul(a[i], b[i]));
    block_reduce_store<1>(acc, partials);
}
// Optional timing of the hinted first round's launches with events on their own stream (measurement only).
struct RoundTimer {
    std::mutex mu;
    bool on = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> ev;
    unsigned long long pairs = 0;
    double bytes = 0;          // algorithmic traffic of the timed launches
};
static RoundTimer g_round_timer;
static RoundTimer g_later_timer;          // the same for the large phase-1 rounds behind the first (k_lookup_round29 / k_lookup_round<false, false>)
static const int g_round_timer_hook = (at_shutdown([] {
    {
        std::lock_guard<std::mutex> lk(g_round_timer.mu);
        for (auto& e : g_round_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
        g_round_timer.ev.clear();
        g_round_timer.on = false;
    }
    {
        std::lock_guard<std::mutex> lk(g_later_timer.mu);
        for (auto& e : g_later_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
        g_later_timer.ev.clear();
        g_later_timer.on = false;
    }
    std::lock_guard<std::mutex> lk(g_eq_mu);
    g_eq_latest.reset();          // the eq table kept for the next job with the same challenges goes back to the allocator
}), 0);
// ZKLLM_FR_LIMBS=32 keeps the round kernels on the 32-bit-limb arithmetic throughout (to compare; the results are the same)
// ZKLLM_LOOKUP_TWO_ROUNDS=0: the first two rounds of a lookup job over int32 queries as two passes (to compare)
static bool two_rounds_on() { static const bool on = [] { const char* e = getenv("ZKLLM_LOOKUP_TWO_ROUNDS"); return !(e && e[0] == '0'); }(); return on; }
static bool limbs29() { static const bool on = [] { const char* e = getenv("ZKLLM_FR_LIMBS"); return !(e && atoi(e) == 32); }(); return on; }
// all rounds of the lookup sumcheck; sums land in job.sums
// A == nullptr with a hint source: 1 / (S + beta) has not been written anywhere; a large first round computes it on
// the fly, anything else writes it out first.
static int lookup_queue(SumJob& job, const Fr* A, const Fr* S, const Fr* B, const Fr* T, const Fr* m, const Fr* E, const Fr& b, const uint32_t* v, size_t D, size_t N, int rounds,
                        const HintSrc* hs = nullptr) {
    hipStream_t st = job.st;
    bool fuse_first = false;
    if (!A) {
        ZK_ARG(hs != nullptr, "lookup sumcheck: neither A nor a hint");
        fuse_first = zk_lookup_ints_suffice(D, N) != 0;       // a phase-1 round that the full-size kernel takes
        if (!fuse_first && hs->S_out) {
            Scratch& Sbuf = job.arena.add(sizeof(Fr) * D);
            if (Sbuf.rc) return Sbuf.rc;
            hipLaunchKernelGGL(k_combine_queries, dim3(cdiv(D, TPB)), dim3(TPB), 0, st, Sbuf.as<Fr>(), hs->hint, hs->S_out, hs->r_mont, D);
            ZK_LAUNCH_CHECK();
            S = Sbuf.as<Fr>();
        }
        if (!fuse_first) {
            Scratch& Abuf = job.arena.add(sizeof(Fr) * D);
            if (Abuf.rc) return Abuf.rc;
            hipLaunchKernelGGL(k_inv_by_hint, dim3(cdiv(D, TPB)), dim3(TPB), 0, st, Abuf.as<Fr>(), S, *hs, D);
            ZK_LAUNCH_CHECK();
            A = Abuf.as<Fr>();
        }
    }
    int n1 = 0;
    while (((size_t)N << n1) < D) ++n1;
    job.rounds = rounds;
    job.per_round = 11;
    job.n1 = n1;
    ZK_ARG(rounds <= FINISH_ROUNDS_MAX, "lookup sumcheck: too many rounds");
    Scratch& sums = job.arena.add(sizeof(Fr) * 11 * rounds);
    // every round keeps its partial sums: one launch sums them all behind the last round
    size_t part_total = 0;
    {
        size_t c = D;
        for (int r = 0; r < rounds; ++r) { c >>= 1; part_total += 11 * (size_t)reduce_grid(c); }
    }
    Scratch& part_all = job.arena.add(sizeof(Fr) * part_total);
    if (sums.rc) return sums.rc;
    if (part_all.rc) return part_all.rc;
    job.sums = sums.as<Fr>();
    ZK_HIP(hipMemsetAsync(sums.p, 0, sizeof(Fr) * 11 * rounds, st));
    FinishRounds fin;
    memset(&fin, 0, sizeof(fin));
    size_t part_at = 0;
    int fin_rounds = 0;              // rounds whose sums come from partials (the rest: the tail kernel's)
    PartSlice part{nullptr};
    const bool eq_prefix = !job.eq_scale.empty();      // every round reads the first table's prefix
    const Fr *cA = A, *cS = S, *cB = B, *cT = T, *cm = m, *cE = E;
    Fr* eqbuf[2] = {nullptr, nullptr};
    size_t cur = D;
    for (int r = 0; r < rounds; ++r) {
        const size_t half = cur >> 1;
        const bool phase2 = r >= n1;
        part.p = part_all.as<Fr>() + part_at;
        if (half <= (size_t)TAIL_HALF && rounds - r <= TAIL_ROUNDS) {
            const int rest = rounds - r;
            Scratch& work = job.arena.add(sizeof(Fr) * 12 * half);
            if (work.rc) return work.rc;
            TailV vs;
            for (int i = 0; i < TAIL_ROUNDS; ++i) vs.v[i] = i < rest ? to_mont(load_fr(v + 8 * (r + i))) : big_zero<8>();
            hipLaunchKernelGGL(k_lookup_tail, dim3(1), dim3(TAIL_T), 0, st, sums.as<Fr>() + (size_t)r * 11, work.as<Fr>(), cA, cS, cB, cT, cm, cE, b, vs, (uint32_t)half,
                               (uint32_t)rest, (uint32_t)(phase2 ? 0 : n1 - r));
            ZK_LAUNCH_CHECK();
            job.tail_from = r;
            break;
        }
        if (r == 0 && !phase2 && fuse_first && hs->hint_ints && limbs29() && two_rounds_on() && n1 >= 2 && rounds >= 2 && (half >> 1) > (size_t)SPLIT_HALF &&
            (half >> 1) <= (size_t)256 * reduce_grid(half >> 1) * TPB) {
            // queries in int32 form, two large phase-1 rounds ahead: both in one pass (k_lookup_first2_29)
            const size_t h2 = half >> 1;
            const unsigned nb2 = reduce_grid(h2);
            Scratch& nx2 = job.arena.add(sizeof(Fr) * h2 * 2);
            if (nx2.rc) return nx2.rc;
            Fr* w2 = nx2.as<Fr>();
            // the third round's eq table goes where the second round would have put it
            Fr* nE3 = nullptr;
            if (r + 2 < rounds && !eq_prefix) {
                Scratch& e = job.arena.add(sizeof(Fr) * 2 * h2);
                if (e.rc) return e.rc;
                eqbuf[0] = e.as<Fr>();
                eqbuf[1] = eqbuf[0] + h2;
                nE3 = eqbuf[1];
            }
            const Fr vm = to_mont(load_fr(v + 8 * r)), vm2 = to_mont(load_fr(v + 8 * (r + 1)));
            const First2Consts cs = first2_consts(b, vm, vm2);
            hipEvent_t t0 = nullptr, t1 = nullptr;
            if (g_round_timer.on) {
                ZK_HIP(hipEventCreate(&t0));
                ZK_HIP(hipEventCreate(&t1));
                ZK_HIP(hipEventRecord(t0, st));
            }
            if (hs->sout_ints) hipLaunchKernelGGL(k_lookup_first2_29<false>, dim3(nb2), dim3(TPB), 0, st, part.as<Fr>(), w2, w2 + h2, cE, b, vm, cs, h2, nE3, *hs);
            else hipLaunchKernelGGL(k_lookup_first2_29<true>, dim3(nb2), dim3(TPB), 0, st, part.as<Fr>(), w2, w2 + h2, cE, b, vm, cs, h2, nE3, *hs);
            if (g_round_timer.on) {
                ZK_HIP(hipEventRecord(t1, st));
                std::lock_guard<std::mutex> lk(g_round_timer.mu);
                g_round_timer.ev.emplace_back(t0, t1);
                g_round_timer.pairs += half;
                // per quad: four queries in int32 form (and their outputs where those are read), two eq weights, two folded values
                // written, half a share of the next table (two more weights read, one written)
                const double q = (hs->sout_ints && !hs->trusted_out) ? 32.0 : 16.0;
                g_round_timer.bytes += (double)h2 * (q + 64.0 + 64.0 + (nE3 ? 48.0 : 0.0));
            }
            ZK_LAUNCH_CHECK();
            if (eq_prefix) job.eq_scale[(size_t)r + 1] = job.eq_scale[(size_t)r];      // the pass forms the second round's weights from the first round's: the same constant
            fin.off[r] = (uint32_t)part_at; fin.nb[r] = nb2; fin.k[r] = 5;
            fin.off[r + 1] = (uint32_t)(part_at + 5 * (size_t)nb2); fin.nb[r + 1] = nb2; fin.k[r + 1] = 5;
            part_at += 10 * (size_t)nb2;
            fin_rounds = r + 2;
            cA = w2; cS = w2 + h2;
            cur = h2;
            if (nE3) cE = nE3;
            ++r;                // two rounds done
            continue;
        }
        Scratch& nx = job.arena.add(sizeof(Fr) * half * (phase2 ? 5 : 2));
        if (nx.rc) return nx.rc;
        Fr* w = nx.as<Fr>();
        // A lane ends with a fixed tail -- its unreduced sums reduced, the workgroup's tree over five or eleven sums: what two to three
        // pairs cost -- so a one-lane-per-pair round with a pair or two per lane pays it per pair.  Those rounds (not the first, whose
        // grid the fused passes choose) take fewer lanes: eight pairs a lane in phase 1, four in phase 2, where the round has them.
        unsigned nb = reduce_grid(half);
        if (half > (size_t)SPLIT_HALF && !(r == 0 && fuse_first)) nb = round_grid(half, phase2 ? 4 : 8);
        const Fr vm = to_mont(load_fr(v + 8 * r));
        // the next round's eq table is written by this round's kernel (ping-pong between two buffers of the job)
        Fr* nE = nullptr;
        if (r + 1 < rounds && !eq_prefix) {
            const size_t nh = half >> 1;
            if (!eqbuf[0]) {
                Scratch& e = job.arena.add(sizeof(Fr) * 2 * (nh ? nh : 1));
                if (e.rc) return e.rc;
                eqbuf[0] = e.as<Fr>();
                eqbuf[1] = eqbuf[0] + (nh ? nh : 1);
            }
            nE = eqbuf[r & 1];
        }
        if (half <= (size_t)SPLIT_HALF) {
            // short round: four lanes per pair (two in phase 1), one task per grid row
            LookupPtrs lp;
            lp.A = cA; lp.S = cS; lp.B = cB; lp.T = cT; lp.m = cm; lp.E = cE; lp.nE = nE;
            lp.nA = w; lp.nS = w + half; lp.nB = w + 2 * half; lp.nT = w + 3 * half; lp.nm = w + 4 * half;
            if (phase2) hipLaunchKernelGGL(k_lookup_round_split<true>, dim3(nb, 4), dim3(TPB), 0, st, part.as<Fr>(), lp, b, vm, half);
            else hipLaunchKernelGGL(k_lookup_round_split<false>, dim3(nb, 2), dim3(TPB), 0, st, part.as<Fr>(), lp, b, vm, half);
        } else if (phase2)
            hipLaunchKernelGGL((k_lookup_round<true, false>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, w + 2 * half, w + 3 * half, w + 4 * half, cA, cS, cB, cT, cm, cE, b, vm, half, nE,
                               HintSrc());
        else if (r == 0 && fuse_first) {
            hipEvent_t t0 = nullptr, t1 = nullptr;
            if (g_round_timer.on) {
                ZK_HIP(hipEventCreate(&t0));
                ZK_HIP(hipEventCreate(&t1));
                ZK_HIP(hipEventRecord(t0, st));
            }
            if (hs->hint_ints && limbs29() && half <= (size_t)512 * nb * TPB)      // queries in int32 form: the common pair in 29-bit limbs
                hipLaunchKernelGGL(k_lookup_first29, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, cE, b, vm, half, nE, *hs);
            else
                hipLaunchKernelGGL((k_lookup_round<false, true>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, (Fr*)nullptr, (Fr*)nullptr, (Fr*)nullptr, (const Fr*)nullptr, cS,
                                   (const Fr*)nullptr, (const Fr*)nullptr, (const Fr*)nullptr, cE, b, vm, half, nE, *hs);
            if (g_round_timer.on) {
                ZK_HIP(hipEventRecord(t1, st));
                std::lock_guard<std::mutex> lk(g_round_timer.mu);
                g_round_timer.ev.emplace_back(t0, t1);
                g_round_timer.pairs += half;
                // per pair: two queries (32 B each; a mapping table's query is two tensors), the eq weight (32 B), two folded values
                // written (64 B), the next round's eq table (16 B)
                // (queries read from their int32 forms: 4 B each)
                const double q = hs->hint_ints ? ((hs->sout_ints && !hs->trusted_out) ? 16.0 : 8.0) : (hs->S_out ? 128.0 : 64.0);      // (trusted outputs are not read)
                g_round_timer.bytes += (double)half * (q + 32.0 + 64.0 + (nE ? 16.0 : 0.0));
            }
        }
        else {
            hipEvent_t t0 = nullptr, t1 = nullptr;
            if (g_later_timer.on) {
                ZK_HIP(hipEventCreate(&t0));
                ZK_HIP(hipEventCreate(&t1));
                ZK_HIP(hipEventRecord(t0, st));
            }
            if (limbs29() && half <= (size_t)256 * nb * TPB)       // 29-bit limbs inside the kernel; its unreduced sums hold 256 pairs per lane
                hipLaunchKernelGGL(k_lookup_round29, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, cA, cS, cE, b, vm, half, nE);
            else
                hipLaunchKernelGGL((k_lookup_round<false, false>), dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, (Fr*)nullptr, (Fr*)nullptr, (Fr*)nullptr, cA, cS, (const Fr*)nullptr,
                                   (const Fr*)nullptr, (const Fr*)nullptr, cE, b, vm, half, nE, HintSrc());
            if (g_later_timer.on) {
                ZK_HIP(hipEventRecord(t1, st));
                std::lock_guard<std::mutex> lk(g_later_timer.mu);
                g_later_timer.ev.emplace_back(t0, t1);
                g_later_timer.pairs += half;
                // per pair: the inverses and queries of both halves (128 B), the eq weight (32 B), two folded values out (64 B), the next eq table (16 B)
                g_later_timer.bytes += (double)half * (128.0 + 32.0 + 64.0 + (nE ? 16.0 : 0.0));
            }
        }
        ZK_LAUNCH_CHECK();
        fin.off[r] = (uint32_t)part_at; fin.nb[r] = nb; fin.k[r] = phase2 ? 11 : 5;
        part_at += (size_t)(phase2 ? 11 : 5) * nb;
        fin_rounds = r + 1;
        cA = w; cS = w + half;
        if (phase2) { cB = w + 2 * half; cT = w + 3 * half; cm = w + 4 * half; }
        cur = half;
        if (nE) cE = nE;
    }
    if (fin_rounds) {
        hipLaunchKernelGGL(k_finish_rounds, dim3(11, fin_rounds), dim3(TPB), 0, st, sums.as<Fr>(), part_all.as<Fr>(), fin, 11u);
        ZK_LAUNCH_CHECK();
    }
    return 0;
}
static int hadamard_queue(SumJob& job, const Fr* const* Xs, int K, const Fr* E, const uint32_t* v, size_t N, const int32_t* const* ints = nullptr) {
    hipStream_t st = job.st;
    int rounds = 0;
    while (((size_t)1 << rounds) < N) ++rounds;
    job.rounds = rounds;
    job.per_round = K + 1;
    ZK_ARG(rounds <= FINISH_ROUNDS_MAX, "Hadamard sumcheck: too many rounds");
    Scratch& sums = job.arena.add(sizeof(Fr) * (K + 1) * rounds);
    size_t part_total = 0;            // every round keeps its partial sums: one launch sums them all behind the last round
    {
        size_t c = N;
        for (int r = 0; r < rounds; ++r) { c >>= 1; part_total += (size_t)(K + 1) * reduce_grid(c); }
    }
    Scratch& part_all = job.arena.add(sizeof(Fr) * part_total);
    if (sums.rc) return sums.rc;
    if (part_all.rc) return part_all.rc;
    job.sums = sums.as<Fr>();
    FinishRounds fin;
    memset(&fin, 0, sizeof(fin));
    size_t part_at = 0;
    int fin_rounds = 0;
    PartSlice part{nullptr};
    const Fr* cur[4];
    for (int i = 0; i < K; ++i) cur[i] = Xs[i];
    const Fr* cE = E;
    Fr* eqbuf[2] = {nullptr, nullptr};
    size_t n = N;
    for (int r = 0; r < rounds; ++r) {
        const size_t half = n >> 1;
        part.p = part_all.as<Fr>() + part_at;
        if (half <= (size_t)TAIL_HALF && rounds - r <= TAIL_ROUNDS) {
            const int rest = rounds - r;
            Scratch& work = job.arena.add(sizeof(Fr) * (K + 1) * half);
            if (work.rc) return work.rc;
            TailV vs;
            for (int i = 0; i < TAIL_ROUNDS; ++i) vs.v[i] = i < rest ? to_mont(load_fr(v + 8 * (r + i))) : big_zero<8>();
            Fr* w = work.as<Fr>();
            Fr* so = sums.as<Fr>() + (size_t)r * (K + 1);
#define HADS_TAIL(KK)                                                                                                                       \
    case KK: {                                                                                                                              \
        PtrPack<KK> p;                                                                                                                      \
        for (int i = 0; i < KK; ++i) { p.in[i] = cur[i]; p.out[i] = w + (size_t)i * half; }                                                  \
        hipLaunchKernelGGL(k_hadamard_tail<KK>, dim3(1), dim3(TAIL_T), 0, st, so, p, w + (size_t)KK * half, cE, vs, (uint32_t)half, (uint32_t)rest); \
        break;                                                                                                                              \
    }
            switch (K) { HADS_TAIL(1) HADS_TAIL(2) HADS_TAIL(3) HADS_TAIL(4) }
#undef HADS_TAIL
            ZK_LAUNCH_CHECK();
            job.tail_from = r;
            break;
        }
        Scratch& nx = job.arena.add(sizeof(Fr) * half * K);
        if (nx.rc) return nx.rc;
        Fr* w = nx.as<Fr>();
        const unsigned nb = reduce_grid(half);
        const Fr vm = to_mont(load_fr(v + 8 * r));
        Fr* nE = nullptr;
        if (r + 1 < rounds && job.eq_scale.empty()) {      // (with eq_scale every round reads the first table's prefix)
            const size_t nh = half >> 1;
            if (!eqbuf[0]) {
                Scratch& e = job.arena.add(sizeof(Fr) * 2 * (nh ? nh : 1));
                if (e.rc) return e.rc;
                eqbuf[0] = e.as<Fr>();
                eqbuf[1] = eqbuf[0] + (nh ? nh : 1);
            }
            nE = eqbuf[r & 1];
        }
#define HADS_ROUND(KK)                                                                                                            \
    case KK: {                                                                                                                    \
        PtrPack<KK> p;                                                                                                            \
        for (int i = 0; i < KK; ++i) { p.in[i] = cur[i]; p.out[i] = w + (size_t)i * half; }                                        \
        hipLaunchKernelGGL(k_hadamard_round<KK>, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), p, cE, vm, half, nE);                  \
        break;                                                                                                                    \
    }
        if (r == 0 && K == 2 && ints && ints[0] && ints[1])
            hipLaunchKernelGGL(k_hadamard_round2_ints, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), ints[0], ints[1], w, w + half, cE, small_fold_consts(vm), half, nE);
        else if (K == 2 && limbs29() && half > (size_t)SPLIT_HALF && half <= (size_t)256 * nb * TPB)      // 29-bit limbs inside the kernel; its unreduced sums hold 256 pairs per lane
            hipLaunchKernelGGL(k_hadamard_round29, dim3(nb), dim3(TPB), 0, st, part.as<Fr>(), w, w + half, cur[0], cur[1], cE, vm, half, nE);
        else
            switch (K) { HADS_ROUND(1) HADS_ROUND(2) HADS_ROUND(3) HADS_ROUND(4) }
#undef HADS_ROUND
        ZK_LAUNCH_CHECK();
        fin.off[r] = (uint32_t)part_at; fin.nb[r] = nb; fin.k[r] = (uint8_t)(K + 1);
        part_at += (size_t)(K + 1) * nb;
        fin_rounds = r + 1;
        for (int i = 0; i < K; ++i) cur[i] = w + (size_t)i * half;
        n = half;
        if (nE) cE = nE;
    }
    if (fin_rounds) {
        hipLaunchKernelGGL(k_finish_rounds, dim3(K + 1, fin_rounds), dim3(TPB), 0, st, sums.as<Fr>(), part_all.as<Fr>(), fin, (uint32_t)(K + 1));
        ZK_LAUNCH_CHECK();
    }
    return 0;
}
// waits for the job's stream and copies its sums (and the extra value) to the host
// a job on a side stream: the copy of its results is queued with it, and collecting waits for that copy only
static int sumjob_queue_results(SumJob& job) {
    const size_t nsum = (size_t)job.rounds * job.per_round;
    int rc = pinned_acquire(&job.host);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(job.host, job.sums, sizeof(Fr) * nsum, hipMemcpyDeviceToHost, job.st));
    if (job.extra) ZK_HIP(hipMemcpyAsync((Fr*)job.host + nsum, job.extra, sizeof(Fr), hipMemcpyDeviceToHost, job.st));
    ZK_HIP(hipEventCreateWithFlags(&job.done, hipEventDisableTiming));
    ZK_HIP(hipEventRecord(job.done, job.st));
    return 0;
}
static int sumjob_collect(SumJob& job, Fr* sums_host, Fr* extra_host) {
    const size_t nsum = (size_t)job.rounds * job.per_round;
    if (job.done) {
        ZK_HIP(hipEventSynchronize(job.done));
        memcpy(sums_host, job.host, sizeof(Fr) * nsum);
        if (job.extra && extra_host) memcpy(extra_host, (Fr*)job.host + nsum, sizeof(Fr));
        return 0;
    }
    void* stage = nullptr;
    int rc = staging(&stage, sizeof(Fr) * (nsum + 1));
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, job.sums, sizeof(Fr) * nsum, hipMemcpyDeviceToHost, job.st));
    if (job.extra) ZK_HIP(hipMemcpyAsync((Fr*)stage + nsum, job.extra, sizeof(Fr), hipMemcpyDeviceToHost, job.st));
    ZK_HIP(hipStreamSynchronize(job.st));
    memcpy(sums_host, stage, sizeof(Fr) * nsum);
    if (job.extra && extra_host) memcpy(extra_host, (Fr*)stage + nsum, sizeof(Fr));
    return 0;
}
// the R corrections of the lookup sums: E carries R, each product one R^-1 (same as zk_lookup_round)
static void lookup_fix_sums(Fr* s, int rounds, int n1) {
    for (int r = 0; r < rounds; ++r)
        for (int i = 0; i < 11; ++i) {
            Fr& x = s[r * 11 + i];
            if (i != 3 && i != 4) x = to_mont(x);
            if (r < n1 && i >= 5) x = big_zero<8>();
        }
}
// the eq table of k challenges for a job on stream st: the latest one when it was built from the same challenges, else a new one
static int shared_eq_get(std::shared_ptr<SharedEq>& out, const uint32_t* u, int k, Arena& arena, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_eq_mu);
    if (g_eq_latest && g_eq_latest->k == k && memcmp(g_eq_latest->key.data(), u, sizeof(uint32_t) * 8 * (size_t)k) == 0) {
        out = g_eq_latest;
        ZK_HIP(hipStreamWaitEvent(st, out->ready, 0));
        return 0;
    }
    std::shared_ptr<SharedEq> e(new SharedEq);
    e->k = k;
    e->key.assign(u, u + 8 * (size_t)k);
    int rc = pool_alloc(&e->p, sizeof(Fr) * ((size_t)1 << k), st);
    if (rc) return rc;
    rc = eq_table_queue((Fr*)e->p, u, k, arena, st);
    if (rc) { (void)hipStreamSynchronize(st); return rc; }
    ZK_HIP(hipEventCreateWithFlags(&e->ready, hipEventDisableTiming));
    ZK_HIP(hipEventRecord(e->ready, st));
    g_eq_latest = e;
    out = e;
    return 0;
}
static int lookup_args_ok(size_t D, size_t N, int rounds) {
    ZK_ARG(D >= 2 && N >= 1 && D % N == 0 && ((D / N) & (D / N - 1)) == 0, "lookup sumcheck: D must be N times a power of two");
    ZK_ARG((D & (D - 1)) == 0, "lookup sumcheck: D must be a power of two");
    ZK_ARG(rounds >= 1 && ((size_t)1 << rounds) <= D && rounds <= 40, "lookup sumcheck: bad round count");
    ZK_ARG(sizeof(Fr) * (11 * (size_t)rounds + 1) <= 65536, "lookup sumcheck: too many rounds for the staging buffer");
    return 0;
}
// puts a new job on one of the library's streams, ordered after everything queued on `caller` so far
static int sumjob_on_side_stream(SumJob& job, hipStream_t caller) {
    job.st = side_stream(1);
    job.arena.st = job.st;
    ZK_ARG(job.st != nullptr, "could not create a stream");
    ZK_HIP(hipEventCreateWithFlags(&job.ready, hipEventDisableTiming));
    ZK_HIP(hipEventRecord(job.ready, caller));
    ZK_HIP(hipStreamWaitEvent(job.st, job.ready, 0));
    pool_note_wait(caller, job.st);
    return 0;
}
// The job's launches: by the launch thread (the caller goes on at once; collecting the job waits for the ticket and reports
// what `queue` returned), or here and now.  queue must not touch memory of the caller's that is only valid during the call.
static int sumjob_launch(SumJob* job, std::function<int()> queue) {
    if (!launcher_enabled()) return queue();
    job->ticket = launcher_submit([job, queue] {
        job->queue_rc = queue();
        if (job->queue_rc) job->queue_err = last_error_text();
    });
    return 0;
}
// before anything of a job is read or released: its launches are on its stream; returns what queuing them returned
static int sumjob_queued(SumJob* job) {
    launcher_wait(job->ticket);
    job->ticket = 0;
    if (job->queue_rc) set_error(job->queue_rc, job->queue_err);
    return job->queue_rc;
}
static void sumjob_abort(SumJob* job) {
    launcher_wait(job->ticket);
    // the job's buffers go back to the allocator: wait for its last use (the whole stream when the job never got as far as its event)
    if (job->done) (void)hipEventSynchronize(job->done);
    else if (job->st) (void)hipStreamSynchronize(job->st);
    job->arena.mark_idle();          // the job's kernels have all finished
    if (job->done) (void)hipEventDestroy(job->done);
    pinned_release(job->host);
    if (job->ready) (void)hipEventDestroy(job->ready);
    delete job;
}

// The whole lookup sumcheck (tLookup_phase1 + tLookup_phase2, tlookup.cu:150-330) queued without a host round trip: the
// fold challenges v (rounds x 8 limbs, in round order) are known up front.  A, S hold D elements, B, T, m hold N
// (D/N a power of two: log2(D/N) phase-1 rounds, then phase-2 rounds), E holds D/2 (Montgomery form).  No input is
// modified.  sums_host: rounds x 11 values ordered as zk_lookup_round orders them.
int zk_lookup_sumcheck(uint32_t* sums_host, const void* A, const void* S, const void* B, const void* T, const void* m, const void* E, const uint32_t* beta,
                       const uint32_t* v, size_t D, size_t N, int rounds, void* stv) {
    int rc = lookup_args_ok(D, N, rounds);
    if (rc) return rc;
    SumJob job;
    job.st = (hipStream_t)stv;
    job.arena.st = job.st;
    rc = lookup_queue(job, (const Fr*)A, (const Fr*)S, (const Fr*)B, (const Fr*)T, (const Fr*)m, (const Fr*)E, load_fr(beta), v, D, N, rounds);
    if (rc) { (void)hipStreamSynchronize(job.st); return rc; }
    rc = sumjob_collect(job, (Fr*)sums_host, nullptr);
    if (rc) return rc;
    lookup_fix_sums((Fr*)sums_host, rounds, job.n1);
    return 0;
}
// The device side of tLookup's proof (tlookup.cu:150-330) as one job beside the caller's stream: A = 1/(S + beta),
// B = 1/(T + beta), <B, m>, the eq table of u_eq (rounds - 1 challenges), then every round.  S: D elements; T, m: N.
// begin returns at once; S, T, m must stay alive and unmodified until end, which waits and delivers <B, m>
// (standard form) and the rounds x 11 sums.  Every handle must be ended exactly once.
// int32 forms (handles of zk_fr_fold_prepare / _new) of the hinted queries, of a mapping table's outputs and of its mapped values
struct LookupInts { const void* queries = nullptr; const void* out = nullptr; const void* mapped = nullptr; };
static int lookup_prove_begin(void** handle, const void* S, const void* T, const void* m, const void* hint, int32_t low, const uint32_t* beta, const uint32_t* u_eq,
                              const uint32_t* v, size_t D, size_t N, int rounds, void* stv, const void* S_out = nullptr, const uint32_t* r = nullptr,
                              const LookupInts* ints = nullptr) {
    ZK_ARG(handle != nullptr, "zk_lookup_prove_begin: null handle");
    int rc = lookup_args_ok(D, N, rounds);
    if (rc) return rc;
    if (ints) {
        const FoldPrepared *q = (const FoldPrepared*)ints->queries, *o = (const FoldPrepared*)ints->out, *mp = (const FoldPrepared*)ints->mapped;
        ZK_ARG(q != nullptr && q->n == D, "lookup sumcheck: the queries' int32 form has another size");
        ZK_ARG(!S_out || (o != nullptr && o->n == D && mp != nullptr && mp->n == N), "lookup sumcheck: a mapping table's int32 forms are missing or of another size");
    }
    SumJob* job = new SumJob;
    rc = sumjob_on_side_stream(*job, (hipStream_t)stv);
    if (rc) { sumjob_abort(job); return rc; }
    // the caller's arrays are only valid during this call: the launches take copies
    const Fr b = load_fr(beta);
    const Fr r_val = r ? load_fr(r) : big_zero<8>();
    const std::vector<uint32_t> u_own(u_eq, u_eq + 8 * (size_t)(rounds - 1)), v_own(v, v + 8 * (size_t)rounds);
    const bool have_ints = ints != nullptr;
    const LookupInts li = ints ? *ints : LookupInts();
    rc = sumjob_launch(job, [=]() -> int {
    int rc = 0;
    const uint32_t *u_eq = u_own.data(), *v = v_own.data();
    const LookupInts* ints = have_ints ? &li : nullptr;
    hipStream_t st = job->st;
    Scratch& B = job->arena.add(sizeof(Fr) * N);
    Scratch& dp = job->arena.add(sizeof(Fr) * (reduce_grid(N) + 1));
    if (B.rc || dp.rc) return B.rc ? B.rc : dp.rc;
    rc = batch_inv_queue(B.as<Fr>(), (const Fr*)T, b, N, job->arena, st);
    const Fr* Aptr = nullptr;
    HintSrc hs;
    if (rc == 0 && hint) {
        Scratch& TB = job->arena.add(sizeof(Fr) * 2 * N);
        if (TB.rc) return TB.rc;
        hipLaunchKernelGGL(k_interleave, dim3(cdiv(N, TPB)), dim3(TPB), 0, st, TB.as<Fr>(), (const Fr*)T, B.as<Fr>(), N);
        hs.TB = TB.as<Fr>(); hs.hint = (const Fr*)hint; hs.low = fr_from_i64((int64_t)low); hs.beta = b; hs.N = (uint32_t)N;
        if (S_out) { hs.S_out = (const Fr*)S_out; hs.r_mont = to_mont(r_val); }
        if (ints) {
            Scratch& want = job->arena.add(sizeof(int32_t) * (N + 1));         // the last slot: n_ok
            if (want.rc) return want.rc;
            const int32_t* mi = S_out ? ((const FoldPrepared*)ints->mapped)->ints : nullptr;
            uint32_t* n_ok = (uint32_t*)(want.as<int32_t>() + N);
            // ZKLLM_LOOKUP_TRUSTED=0: no entry counts as checked and no output as gathered from the table -- every query goes
            // through its own comparison (to compare the two paths)
            static const bool trust = [] { const char* e = getenv("ZKLLM_LOOKUP_TRUSTED"); return !(e && e[0] == '0'); }();
            hipLaunchKernelGGL(k_u32_set, dim3(1), dim3(64), 0, st, n_ok, trust ? 0xFFFFFFFFu : 0u);      // a kernel, not a memset node: callers may capture this
            hipLaunchKernelGGL(k_lookup_ints_check, dim3(cdiv(N, TPB)), dim3(TPB), 0, st, want.as<int32_t>(), n_ok, TB.as<Fr>(), mi, hs.r_mont, low, (uint32_t)N);
            hs.n_ok = n_ok;
            job->n_ok_dev = n_ok;
            job->n_table = (uint32_t)N;
            if (S_out) {
                const FoldPrepared *q = (const FoldPrepared*)ints->queries, *o = (const FoldPrepared*)ints->out, *mp = (const FoldPrepared*)ints->mapped;
                hs.trusted_out = trust && o->src_queries != 0 && o->src_queries == q->id && o->src_table == mp->id && o->src_low == low;
            }
            hs.hint_ints = ((const FoldPrepared*)ints->queries)->ints;
            hs.sout_ints = S_out ? ((const FoldPrepared*)ints->out)->ints : nullptr;
            hs.want = want.as<int32_t>();
            hs.low_int = low;
        }
    } else if (rc == 0) {
        Scratch& A = job->arena.add(sizeof(Fr) * D);
        rc = A.rc;
        if (rc == 0) rc = batch_inv_queue(A.as<Fr>(), (const Fr*)S, b, D, job->arena, st);
        Aptr = A.as<Fr>();
    }
    if (rc) return rc;
    const unsigned nb = reduce_grid(N);
    hipLaunchKernelGGL(k_dot_part, dim3(nb), dim3(TPB), 0, st, dp.as<Fr>() + 1, B.as<Fr>(), (const Fr*)m, N);
    hipLaunchKernelGGL(k_finish, dim3(1), dim3(TPB), 0, st, dp.as<Fr>(), dp.as<Fr>() + 1, nb);
    job->extra = dp.as<Fr>();
    rc = shared_eq_get(job->eq, u_eq, rounds - 1, job->arena, st);
    if (rc) return rc;
    if (eq_prefix_on()) (void)eq_prefix_scales(job->eq_scale, u_eq, rounds);
    rc = lookup_queue(*job, Aptr, (const Fr*)S, B.as<Fr>(), (const Fr*)T, (const Fr*)m, (const Fr*)job->eq->p, b, v, D, N, rounds, hint ? &hs : nullptr);
    if (rc == 0) rc = sumjob_queue_results(*job);
    return rc;
    });
    if (rc) { sumjob_abort(job); return rc; }
    *handle = job;
    return 0;
}
int zk_lookup_prove_begin(void** handle, const void* S, const void* T, const void* m, const uint32_t* beta, const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N,
                          int rounds, void* stv) {
    return lookup_prove_begin(handle, S, T, m, nullptr, 0, beta, u_eq, v, D, N, rounds, stv);
}
// The same for queries that are expected to be table entries, with a hint where: query i should equal T[hint[i] - low]
// (hint: D field elements -- for a range table, the looked-up values themselves).  The results are those of
// zk_lookup_prove_begin for every input; where the hint holds, 1/(S[i] + beta) is read from the table's inverses.
int zk_lookup_prove_begin_hinted(void** handle, const void* S, const void* T, const void* m, const void* hint, int32_t low, const uint32_t* beta, const uint32_t* u_eq,
                                 const uint32_t* v, size_t D, size_t N, int rounds, void* stv) {
    ZK_ARG(hint != nullptr, "zk_lookup_prove_begin_hinted: null hint");
    return lookup_prove_begin(handle, S, T, m, hint, low, beta, u_eq, v, D, N, rounds, stv);
}
// The same for a mapping table's combined lookup (tlookup.cu:517-518): query i is S_in[i] + r * S_out[i], expected at
// T[S_in[i] - low] with T the combined table.  The combined queries are never written out when the job is large enough for
// its first round to form them on the fly.
int zk_lookup_prove_begin_mapped(void** handle, const void* S_in, const void* S_out, const uint32_t* r, const void* T, const void* m, int32_t low, const uint32_t* beta,
                                 const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N, int rounds, void* stv) {
    ZK_ARG(S_in != nullptr && S_out != nullptr && r != nullptr, "zk_lookup_prove_begin_mapped: null queries or challenge");
    return lookup_prove_begin(handle, nullptr, T, m, S_in, low, beta, u_eq, v, D, N, rounds, stv, S_out, r);
}
// 1 when a job of this shape takes its queries from their int32 forms alone (its first round is the fused one): the
// field-element tensor given beside them is then never read
int zk_lookup_ints_suffice(size_t D, size_t N) { return (D > N && (D >> 1) > (size_t)SPLIT_HALF) ? 1 : 0; }
int zk_lookup_prove_begin_hinted_ints(void** handle, const void* S, const void* S_prepared, const void* T, const void* m, int32_t low, const uint32_t* beta,
                                      const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N, int rounds, void* stv) {
    ZK_ARG(S != nullptr && S_prepared != nullptr, "zk_lookup_prove_begin_hinted_ints: null queries");
    LookupInts li;
    li.queries = S_prepared;
    return lookup_prove_begin(handle, S, T, m, S, low, beta, u_eq, v, D, N, rounds, stv, nullptr, nullptr, &li);
}
int zk_lookup_prove_begin_mapped_ints(void** handle, const void* S_in, const void* S_in_prepared, const void* S_out, const void* S_out_prepared, const void* mapped_prepared,
                                      const uint32_t* r, const void* T, const void* m, int32_t low, const uint32_t* beta, const uint32_t* u_eq, const uint32_t* v, size_t D,
                                      size_t N, int rounds, void* stv) {
    ZK_ARG(S_in != nullptr && S_out != nullptr && r != nullptr, "zk_lookup_prove_begin_mapped_ints: null queries or challenge");
    ZK_ARG(S_in_prepared != nullptr && S_out_prepared != nullptr && mapped_prepared != nullptr, "zk_lookup_prove_begin_mapped_ints: null int32 form");
    LookupInts li;
    li.queries = S_in_prepared; li.out = S_out_prepared; li.mapped = mapped_prepared;
    return lookup_prove_begin(handle, nullptr, T, m, S_in, low, beta, u_eq, v, D, N, rounds, stv, S_out, r, &li);
}
// what the last collected lookup job over int32 forms found: how many leading table entries were what the integers say
// (the queries that name one of them took the first round's short path), and the table's size; 0, 0 when that job had no int32 forms
static uint32_t g_last_n_ok = 0, g_last_n_table = 0;
int zk_lookup_last_job_consistent_entries(uint32_t* n_ok, uint32_t* n_table) {
    if (n_ok) *n_ok = g_last_n_ok;
    if (n_table) *n_table = g_last_n_table;
    return 0;
}
int zk_lookup_prove_end(void* handle, uint32_t* bm_host, uint32_t* sums_host) {
    ZK_ARG(handle != nullptr, "zk_lookup_prove_end: null handle");
    SumJob* job = (SumJob*)handle;
    Fr bm = big_zero<8>();
    int rc = sumjob_queued(job);
    if (rc) { sumjob_abort(job); return rc; }
    rc = sumjob_collect(*job, (Fr*)sums_host, &bm);
    g_last_n_ok = g_last_n_table = 0;
    if (!rc && job->n_ok_dev) {          // the job's kernels have finished
        uint32_t v = 0;
        if (hipMemcpy(&v, job->n_ok_dev, sizeof(uint32_t), hipMemcpyDeviceToHost) == hipSuccess) { g_last_n_ok = v < job->n_table ? v : job->n_table; g_last_n_table = job->n_table; }
    }
    if (!rc) {
        eq_prefix_apply(*job, (Fr*)sums_host, 0x0E7u);      // sums 0..2 and 5..7: sums 3, 4 and 8..10 carry no eq weight
        lookup_fix_sums((Fr*)sums_host, job->rounds, job->n1);
        bm = to_mont(bm);          // the products carried R^-1
        memcpy(bm_host, &bm, sizeof(Fr));
    }
    sumjob_abort(job);
    return rc;
}
// Measurement: time every launch of the hinted first round (k_lookup_round<false, true>) between begin and read, with events
// on the launch stream.  bytes: the algorithmic traffic of those launches.
static void round_timer_begin(RoundTimer& T) {
    std::lock_guard<std::mutex> lk(T.mu);
    for (auto& e : T.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    T.ev.clear();
    T.pairs = 0;
    T.bytes = 0;
    T.on = true;
}
static int round_timer_read(RoundTimer& T, double* total_ms, unsigned long long* launches, unsigned long long* pairs, double* bytes) {
    std::lock_guard<std::mutex> lk(T.mu);
    T.on = false;
    double tot = 0;
    for (auto& e : T.ev) {
        ZK_HIP(hipEventSynchronize(e.second));
        float ms = 0;
        ZK_HIP(hipEventElapsedTime(&ms, e.first, e.second));
        tot += ms;
    }
    *total_ms = tot;
    *launches = T.ev.size();
    *pairs = T.pairs;
    *bytes = T.bytes;
    for (auto& e : T.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    T.ev.clear();
    return 0;
}
int zk_prof_lookup_begin(void) {
    round_timer_begin(g_round_timer);
    round_timer_begin(g_later_timer);
    return 0;
}
int zk_prof_lookup_read(double* total_ms, unsigned long long* launches, unsigned long long* pairs, double* bytes) {
    return round_timer_read(g_round_timer, total_ms, launches, pairs, bytes);
}
// the large phase-1 rounds behind the first (one lane per pair: k_lookup_round29 or k_lookup_round<false, false>) since zk_prof_lookup_begin
int zk_prof_lookup_later_read(double* total_ms, unsigned long long* launches, unsigned long long* pairs, double* bytes) {
    return round_timer_read(g_later_timer, total_ms, launches, pairs, bytes);
}
// The whole multi-Hadamard sumcheck (proof.cu:191-241) queued without a host round trip.  Xs: K tensors of N elements
// (N a power of two), E: N/2 elements (Montgomery form), v: log2(N) fold challenges in round order.  coefs_host:
// log2(N) x (K+1) coefficients.  No input is modified.
int zk_hadamard_sumcheck(uint32_t* coefs_host, const void* const* Xs, int K, const void* E, const uint32_t* v, size_t N, void* stv) {
    ZK_ARG(K >= 1 && K <= 4, "zk_hadamard_sumcheck: K must be 1..4");
    ZK_ARG(N >= 2 && (N & (N - 1)) == 0, "zk_hadamard_sumcheck: N must be a power of two >= 2");
    SumJob job;
    job.st = (hipStream_t)stv;
    job.arena.st = job.st;
    int rc = hadamard_queue(job, (const Fr* const*)Xs, K, (const Fr*)E, v, N);
    if (rc) { (void)hipStreamSynchronize(job.st); return rc; }
    return sumjob_collect(job, (Fr*)coefs_host, nullptr);
}
// The same beside the caller's stream, eq table of u_eq (log2(N) - 1 challenges) included.  Xs must stay alive and
// unmodified until end; every handle must be ended exactly once.
// 1 when a Hadamard job of K tensors of N elements that all carry int32 forms reads nothing but those forms
int zk_hadamard_ints_suffice(int K, size_t N) {
    if (K != 2 || N < 2 || (N & (N - 1))) return 0;
    int rounds = 0;
    while (((size_t)1 << rounds) < N) ++rounds;
    return ((N >> 1) <= (size_t)TAIL_HALF && rounds <= TAIL_ROUNDS) ? 0 : 1;      // a job that is all tail reads the field elements
}
int zk_hadamard_prove_begin(void** handle, const void* const* Xs, int K, const uint32_t* u_eq, const uint32_t* v, size_t N, void* stv) {
    return zk_hadamard_prove_begin_ints(handle, Xs, nullptr, K, u_eq, v, N, stv);
}
int zk_hadamard_prove_begin_ints(void** handle, const void* const* Xs, const void* const* prepareds, int K, const uint32_t* u_eq, const uint32_t* v, size_t N, void* stv) {
    ZK_ARG(handle != nullptr, "zk_hadamard_prove_begin: null handle");
    const int32_t* ints[4] = {nullptr, nullptr, nullptr, nullptr};
    if (prepareds)
        for (int i = 0; i < K && i < 4; ++i)
            if (const FoldPrepared* fp = (const FoldPrepared*)prepareds[i]) {
                ZK_ARG(fp->n == N, "zk_hadamard_prove_begin_ints: an int32 form of another size");
                ints[i] = fp->ints;
            }
    ZK_ARG(K >= 1 && K <= 4, "zk_hadamard_prove_begin: K must be 1..4");
    ZK_ARG(N >= 2 && (N & (N - 1)) == 0, "zk_hadamard_prove_begin: N must be a power of two >= 2");
    SumJob* job = new SumJob;
    int rc = sumjob_on_side_stream(*job, (hipStream_t)stv);
    if (rc) { sumjob_abort(job); return rc; }
    int k = 0;
    while (((size_t)1 << k) < N) ++k;
    // the caller's arrays are only valid during this call: the launches take copies
    const std::vector<uint32_t> u_own(u_eq, u_eq + 8 * (size_t)(k - 1)), v_own(v, v + 8 * (size_t)k);
    const std::vector<const Fr*> xs_own((const Fr* const*)Xs, (const Fr* const*)Xs + K);
    const std::vector<const int32_t*> ints_own(ints, ints + 4);
    const bool have_ints = prepareds != nullptr;
    rc = sumjob_launch(job, [=]() -> int {
        int rc = shared_eq_get(job->eq, u_own.data(), k - 1, job->arena, job->st);
        if (rc) return rc;
        if (eq_prefix_on()) (void)eq_prefix_scales(job->eq_scale, u_own.data(), k);
        rc = hadamard_queue(*job, xs_own.data(), K, (const Fr*)job->eq->p, v_own.data(), N, have_ints ? ints_own.data() : nullptr);
        if (rc == 0) rc = sumjob_queue_results(*job);
        return rc;
    });
    if (rc) { sumjob_abort(job); return rc; }
    *handle = job;
    return 0;
}
int zk_hadamard_prove_end(void* handle, uint32_t* coefs_host) {
    ZK_ARG(handle != nullptr, "zk_hadamard_prove_end: null handle");
    SumJob* job = (SumJob*)handle;
    int rc = sumjob_queued(job);
    if (rc) { sumjob_abort(job); return rc; }
    rc = sumjob_collect(*job, (Fr*)coefs_host, nullptr);
    if (!rc) eq_prefix_apply(*job, (Fr*)coefs_host, 0xFFFFFFFFu);      // every coefficient is eq-weighted
    sumjob_abort(job);
    return rc;
}
// hadamard_product_sumcheck (proof.cu:66-109): k rounds over a, b of n elements (2^(k-1) < n <= 2^k), evaluation
// challenges u and fold challenges v, both in the order the reference consumes them (first challenge first).
// proof_host: 3k + 2 values -- per round the three evaluated terms, then the fully folded a and b.  Neither input is modified.
// the launches of hadamard_product_sumcheck on st, its buffers from `arena`; *sums_out: the 3k + 2 values on the device
static int hp_sumcheck_queue(Fr** sums_out, Arena& arena, const void* a, const void* b, const uint32_t* u, const uint32_t* v, size_t n, int k, hipStream_t st) {
    const size_t half = (n + 1) / 2, etab = (size_t)1 << (k - 1);
    Scratch& E = arena.add(sizeof(Fr) * (etab + etab / 2 + 1));          // eq tables, ping-pong
    Scratch& W = arena.add(sizeof(Fr) * 2 * (half + (half + 1) / 2 + 1));   // folded a, b, ping-pong
    size_t part_total = 0;            // every round keeps its partial sums: one launch sums them all behind the last round
    {
        size_t c = n;
        for (int r = 0; r < k; ++r) { c = (c + 1) / 2; part_total += 3 * (size_t)reduce_grid(c); }
    }
    Scratch& part = arena.add(sizeof(Fr) * part_total);
    Scratch& sums = arena.add(sizeof(Fr) * (3 * (size_t)k + 2));
    if (E.rc || W.rc || part.rc || sums.rc) return E.rc ? E.rc : (W.rc ? W.rc : (part.rc ? part.rc : sums.rc));
    FinishRounds fin;
    memset(&fin, 0, sizeof(fin));
    size_t part_at = 0;
    int rc = eq_table_queue(E.as<Fr>(), u + 8, k - 1, arena, st);
    if (rc) return rc;
    Fr* ebuf[2] = {E.as<Fr>(), E.as<Fr>() + etab};
    Fr* wa[2] = {W.as<Fr>(), W.as<Fr>() + half};
    Fr* wb[2] = {wa[1] + (half + 1) / 2 + 1, nullptr};
    wb[1] = wb[0] + half;
    const Fr *ca = (const Fr*)a, *cb = (const Fr*)b, *ce = ebuf[0];
    size_t cur = n, ecur = etab;
    for (int r = 0; r < k; ++r) {
        const size_t out = (cur + 1) / 2;
        const unsigned nb = reduce_grid(out);
        hipLaunchKernelGGL(k_hp_round, dim3(nb), dim3(TPB), 0, st, part.as<Fr>() + part_at, wa[r & 1], wb[r & 1], ebuf[(r + 1) & 1], ca, cb, ce, to_mont(load_fr(v + 8 * r)), cur, out, ecur / 2);
        ZK_LAUNCH_CHECK();
        fin.off[r] = (uint32_t)part_at; fin.nb[r] = nb; fin.k[r] = 3;
        part_at += 3 * (size_t)nb;
        ca = wa[r & 1]; cb = wb[r & 1]; ce = ebuf[(r + 1) & 1];
        cur = out;
        ecur /= 2;
    }
    hipLaunchKernelGGL(k_finish_rounds, dim3(3, k), dim3(TPB), 0, st, sums.as<Fr>(), part.as<Fr>(), fin, 3u);
    ZK_LAUNCH_CHECK();
    ZK_HIP(hipMemcpyAsync(sums.as<Fr>() + 3 * (size_t)k, ca, sizeof(Fr), hipMemcpyDeviceToDevice, st));
    ZK_HIP(hipMemcpyAsync(sums.as<Fr>() + 3 * (size_t)k + 1, cb, sizeof(Fr), hipMemcpyDeviceToDevice, st));
    *sums_out = sums.as<Fr>();
    return 0;
}
int zk_hadamard_product_sumcheck(uint32_t* proof_host, const void* a, const void* b, const uint32_t* u, const uint32_t* v, size_t n, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(k >= 1 && k <= 30 && n <= ((size_t)1 << k) && n > ((size_t)1 << (k - 1)), "zk_hadamard_product_sumcheck: n does not match the number of challenges");
    ZK_ARG(sizeof(Fr) * (3 * (size_t)k + 2) <= 65536, "zk_hadamard_product_sumcheck: too many rounds for the staging buffer");
    Arena arena(st);
    Fr* sums = nullptr;
    int rc = hp_sumcheck_queue(&sums, arena, a, b, u, v, n, k, st);
    if (rc) { (void)hipStreamSynchronize(st); return rc; }
    void* stage = nullptr;
    rc = staging(&stage, sizeof(Fr) * (3 * (size_t)k + 2));
    if (rc) { (void)hipStreamSynchronize(st); return rc; }
    ZK_HIP(hipMemcpyAsync(stage, sums, sizeof(Fr) * (3 * (size_t)k + 2), hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    memcpy(proof_host, stage, sizeof(Fr) * (3 * (size_t)k + 2));
    return 0;
}
// The same in two halves: begin queues the rounds on a stream of the library's own, behind everything queued on `stream` so
// far, and returns at once; a and b must stay alive and unmodified until end, which waits and delivers the 3k + 2 values.
int zk_hadamard_product_sumcheck_begin(void** handle, const void* a, const void* b, const uint32_t* u, const uint32_t* v, size_t n, int k, void* stv) {
    ZK_ARG(handle != nullptr, "zk_hadamard_product_sumcheck_begin: null handle");
    ZK_ARG(k >= 1 && k <= 30 && n <= ((size_t)1 << k) && n > ((size_t)1 << (k - 1)), "zk_hadamard_product_sumcheck: n does not match the number of challenges");
    ZK_ARG(sizeof(Fr) * (3 * (size_t)k + 2) <= 65536, "zk_hadamard_product_sumcheck: too many rounds for the staging buffer");
    SumJob* job = new SumJob;
    int rc = sumjob_on_side_stream(*job, (hipStream_t)stv);
    if (rc) { sumjob_abort(job); return rc; }
    // the caller's arrays are only valid during this call: the launches take copies
    const std::vector<uint32_t> u_own(u, u + 8 * (size_t)k), v_own(v, v + 8 * (size_t)k);
    job->rounds = 1;
    job->per_round = 3 * k + 2;
    rc = sumjob_launch(job, [=]() -> int {
        int rc = hp_sumcheck_queue(&job->sums, job->arena, a, b, u_own.data(), v_own.data(), n, k, job->st);
        if (rc == 0) rc = sumjob_queue_results(*job);
        return rc;
    });
    if (rc) { sumjob_abort(job); return rc; }
    *handle = job;
    return 0;
}
int zk_hadamard_product_sumcheck_end(void* handle, uint32_t* proof_host) {
    ZK_ARG(handle != nullptr, "zk_hadamard_product_sumcheck_end: null handle");
    SumJob* job = (SumJob*)handle;
    int rc = sumjob_queued(job);
    if (rc) { sumjob_abort(job); return rc; }
    rc = sumjob_collect(*job, (Fr*)proof_host, nullptr);
    sumjob_abort(job);
    return rc;
}
int zk_rescale(void* out, void* rem, const void* in, uint32_t scaling_factor, size_t n, void* st) {
    ZK_ARG(scaling_factor >= 1, "zk_rescale: scaling factor is 0");
    LAUNCH1D(k_rescale, n, st, (Fr*)out, (Fr*)rem, (int32_t*)nullptr, (const Fr*)in, (int64_t)scaling_factor, n);
    return 0;
}
int zk_rescale_ints(void* out, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* st) {
    ZK_ARG(scaling_factor >= 1, "zk_rescale: scaling factor is 0");
    ZK_ARG(rem != nullptr || rem_ints != nullptr, "zk_rescale_ints: the remainders need at least one form");
    LAUNCH1D(k_rescale, n, st, (Fr*)out, (Fr*)rem, (int32_t*)rem_ints, (const Fr*)in, (int64_t)scaling_factor, n);
    return 0;
}
int zk_rescale_ints_both(void* out, void* out_ints, int* out_fits_host, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(scaling_factor >= 1, "zk_rescale: scaling factor is 0");
    ZK_ARG(out_ints != nullptr && out_fits_host != nullptr, "zk_rescale_ints_both: null argument");
    ZK_ARG(rem != nullptr || rem_ints != nullptr, "zk_rescale_ints_both: the remainders need at least one form");
    *out_fits_host = 1;
    if (n == 0) return 0;
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    LAUNCH1D(k_rescale, n, st, (Fr*)out, (Fr*)rem, (int32_t*)rem_ints, (const Fr*)in, (int64_t)scaling_factor, n, (int32_t*)out_ints, flag.as<uint32_t>());
    uint32_t f = 0;
    int rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    *out_fits_host = f ? 0 : 1;
    return 0;
}
// the same without the round trip: *bad_flag_dev (4 bytes of device memory) is cleared and then raised by the kernel when a
// rescaled value does not fit; the caller reads it once the kernel is through, whenever that suits it
int zk_rescale_ints_both_flag(void* out, void* out_ints, void* bad_flag_dev, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(scaling_factor >= 1, "zk_rescale: scaling factor is 0");
    ZK_ARG(out_ints != nullptr && bad_flag_dev != nullptr, "zk_rescale_ints_both_flag: null argument");
    ZK_ARG(rem != nullptr || rem_ints != nullptr, "zk_rescale_ints_both_flag: the remainders need at least one form");
    ZK_HIP(hipMemsetAsync(bad_flag_dev, 0, 4, st));
    if (n == 0) return 0;
    LAUNCH1D(k_rescale, n, st, (Fr*)out, (Fr*)rem, (int32_t*)rem_ints, (const Fr*)in, (int64_t)scaling_factor, n, (int32_t*)out_ints, (uint32_t*)bad_flag_dev);
    return 0;
}
int zk_i32_fill(void* dst, int32_t value, size_t n, void* st) {
    LAUNCH1D(k_i32_fill, n, st, (int32_t*)dst, value, n);
    return 0;
}
int zk_relu_decomp(void* res, void* sign, void* mag, void* rem, const void* in, uint32_t scaling_factor, size_t n, void* st) {
    ZK_ARG(scaling_factor >= 1, "zk_relu_decomp: scaling factor is 0");
    LAUNCH1D(k_relu_decomp, n, st, (Fr*)res, (Fr*)sign, (Fr*)mag, (Fr*)rem, (const Fr*)in, (int64_t)scaling_factor, n);
    return 0;
}
int zk_softmax_shift(void* shift, void* out_shifted, const void* X, uint32_t rows, uint32_t cols, double scale, void* st) {
    if (rows == 0) return 0;
    ZK_ARG(cols >= 1 && scale > 0.0, "zk_softmax_shift: bad shape or scale");
    hipLaunchKernelGGL(k_softmax_shift, dim3(cdiv(rows, TPB / 64)), dim3(TPB), 0, (hipStream_t)st, (Fr*)shift, (Fr*)out_shifted, (const Fr*)X, rows, cols, scale, PlanePtrs(),
                       IntPlanePtrs(), (uint32_t*)nullptr, U32Pack8(), 0);
    ZK_LAUNCH_CHECK();
    return 0;
}
static int softmax_shift_decompose(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X, const void* X64, uint32_t rows, uint32_t cols,
                                   double scale, const uint32_t* bs_host, int K, void* stv);
int zk_softmax_shift_decompose(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X, uint32_t rows, uint32_t cols, double scale,
                               const uint32_t* bs_host, int K, void* stv) {
    return softmax_shift_decompose(shift, out_shifted, planes, int_planes, X, nullptr, rows, cols, scale, bs_host, K, stv);
}
// the same over scores given as 64-bit integers (rows * cols int64 on the device, zk_fr_matmul_batched_i64)
int zk_softmax_shift_decompose_i64(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X64, uint32_t rows, uint32_t cols, double scale,
                                   const uint32_t* bs_host, int K, void* stv) {
    ZK_ARG(X64 != nullptr, "zk_softmax_shift_decompose_i64: null scores");
    return softmax_shift_decompose(shift, out_shifted, planes, int_planes, nullptr, X64, rows, cols, scale, bs_host, K, stv);
}
static int softmax_shift_decompose(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X, const void* X64, uint32_t rows, uint32_t cols,
                                   double scale, const uint32_t* bs_host, int K, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (rows == 0) return 0;
    ZK_ARG(cols >= 1 && scale > 0.0, "zk_softmax_shift: bad shape or scale");
    ZK_ARG(K >= 1 && K <= 8, "zk_softmax_decompose: K must be 1..8");
    U32Pack8 bs;
    for (int i = 0; i < 8; ++i) bs.v[i] = i < K ? bs_host[i] : 1u;
    for (int i = 0; i < K; ++i) ZK_ARG(bs.v[i] >= 1, "zk_softmax_decompose: zero radix");
    PlanePtrs pp;
    IntPlanePtrs ip;
    for (int i = 0; i < 8; ++i) { pp.p[i] = i < K ? (Fr*)planes[i] : nullptr; ip.p[i] = (int_planes && i < K) ? (int32_t*)int_planes[i] : nullptr; }
    for (int i = 0; i < K; ++i) ZK_ARG(pp.p[i] != nullptr || ip.p[i] != nullptr, "zk_softmax_decompose: a digit with neither plane");
    for (int i = 0; i < K; ++i) ZK_ARG(!ip.p[i] || bs.v[i] <= 0x80000000u, "zk_softmax_decompose_ints: a radix above 2^31 has no int32 plane");
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    hipLaunchKernelGGL(k_softmax_shift, dim3(cdiv(rows, TPB / 64)), dim3(TPB), 0, st, (Fr*)shift, (Fr*)out_shifted, (const Fr*)X, rows, cols, scale, pp, ip, flag.as<uint32_t>(), bs, K,
                       (const int64_t*)X64);
    ZK_LAUNCH_CHECK();
    uint32_t f = 0;
    int rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    ZK_ARG(f == 0, "softmax: a shifted score is positive or exceeds the digit radices");
    return 0;
}
int zk_softmax_table(void* table, double log_theta, double step, uint32_t len, void* st) {
    LAUNCH1D(k_softmax_table, len, st, (Fr*)table, log_theta, step, len);
    return 0;
}
// planes: K device tensors of n elements, plane k = digit k of -X in the mixed radix bs_host[0..K)
int zk_softmax_decompose(void* const* planes, const void* X_shifted, const uint32_t* bs_host, int K, size_t n, void* stv) {
    return zk_softmax_decompose_ints(planes, nullptr, X_shifted, bs_host, K, n, stv);
}
int zk_softmax_decompose_ints(void* const* planes, void* const* int_planes, const void* X_shifted, const uint32_t* bs_host, int K, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(K >= 1 && K <= 8, "zk_softmax_decompose: K must be 1..8");
    if (n == 0) return 0;
    U32Pack8 bs;
    for (int i = 0; i < 8; ++i) bs.v[i] = i < K ? bs_host[i] : 1u;
    for (int i = 0; i < K; ++i) ZK_ARG(bs.v[i] >= 1, "zk_softmax_decompose: zero radix");
    Scratch flag(4, st);
    if (flag.rc) return flag.rc;
    ZK_HIP(hipMemsetAsync(flag.p, 0, 4, st));
    PlanePtrs pp;
    for (int i = 0; i < 8; ++i) pp.p[i] = i < K ? (Fr*)planes[i] : nullptr;
    for (int i = 0; i < K; ++i) ZK_ARG(pp.p[i] != nullptr, "zk_softmax_decompose: null plane");
    IntPlanePtrs ip;
    for (int i = 0; i < 8; ++i) ip.p[i] = (int_planes && i < K) ? (int32_t*)int_planes[i] : nullptr;
    for (int i = 0; i < K; ++i) ZK_ARG(!ip.p[i] || bs.v[i] <= 0x80000000u, "zk_softmax_decompose_ints: a radix above 2^31 has no int32 plane");
    LAUNCH1D(k_softmax_decompose, n, st, pp, ip, flag.as<uint32_t>(), (const Fr*)X_shifted, bs, K, n);
    uint32_t f = 0;
    int rc = read_flag(flag.as<uint32_t>(), &f, st);
    if (rc) return rc;
    ZK_ARG(f == 0, "softmax: a shifted score is positive or exceeds the digit radices");
    return 0;
}

}  // extern "C"

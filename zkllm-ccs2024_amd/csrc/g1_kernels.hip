// G1 tensor kernels and the Pedersen commitment for gfx950.
//
// Points are Jacobian (x,y,z) over Fp in Montgomery form, 144 B each -- the reference's
// G1Jacobian_t layout (bls12-381.cuh:429-433).  Replaces g1-tensor.cu:61-625 (elementwise ops,
// sum, row-wise sum, scalar multiplication, G1 multilinear fold) and commitment.cu:22-129
// (commit, commit_int, me_open_step).
//
// commit_int is a fixed-base windowed multi-scalar multiplication: the generators are shared by
// every row of the committed matrix, so their signed-window multiples d*2^(cw)*G_j are built once
// (affine, batch-normalised) and each row is a run of mixed additions out of that table -- no
// per-pair doublings and no materialised m*n temporary (the reference writes 144 B per pair).
// All of it is VALU integer work on 12-limb Fp; results equal the reference's as group elements
// (a Jacobian triple depends on the order of additions, so bytes are compared after normalising).
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>
#include "fq29.hpp"
#include "rt.hpp"
#include "../../include/zkllm_hip.h"

using namespace zk;

static constexpr int GT = 64;   // threads per workgroup for point kernels (one wave; ~200 VGPRs per lane)

// ---- elementwise -------------------------------------------------------------------------------------
__global__ void __launch_bounds__(GT) k_g1_fill(G1Jac* __restrict__ out, const G1Jac p, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i < n) out[i] = p;
}
__global__ void __launch_bounds__(GT) k_g1_neg(G1Jac* __restrict__ out, const G1Jac* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i < n) out[i] = g1_neg(a[i]);
}
__global__ void __launch_bounds__(GT) k_g1aff_neg(G1Affine* __restrict__ out, const G1Affine* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i < n) out[i] = g1_neg(a[i]);
}
__global__ void __launch_bounds__(GT) k_g1aff_to_jac(G1Jac* __restrict__ out, const G1Affine* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= n) return;
    G1Jac r; r.x = a[i].x; r.y = a[i].y; r.z = big_one_mont<12>();
    out[i] = r;
}
// out = a (+/-) b ; nb == n elementwise, nb == 1 broadcast
__global__ void __launch_bounds__(GT) k_g1_add(G1Jac* __restrict__ out, const G1Jac* __restrict__ a, const G1Jac* __restrict__ b, size_t n, size_t nb, int negate) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= n) return;
    G1Jac q = b[nb == 1 ? 0 : i];
    if (negate) q = g1_neg(q);
    out[i] = g1_add(a[i], q);
}
__global__ void __launch_bounds__(GT) k_g1_madd(G1Jac* __restrict__ out, const G1Jac* __restrict__ a, const G1Affine* __restrict__ b, size_t n, size_t nb, int negate) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= n) return;
    G1Affine q = b[nb == 1 ? 0 : i];
    if (negate) q = g1_neg(q);
    out[i] = g1_add_mixed(a[i], q);
}
// out[i] = [s[i]] g[i % ng]   (G1_jacobian_elementwise_mul / _mul_broadcast, g1-tensor.cu:456-482)
__global__ void __launch_bounds__(GT) k_g1_scalar_mul(G1Jac* __restrict__ out, const G1Jac* __restrict__ g, const Fr* __restrict__ s, size_t ng, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i < n) out[i] = g1_mul(g[i % ng], s[i]);
}

// ---- reductions ------------------------------------------------------------------------------------------
// LDS tree over the GT lanes of a workgroup; lane 0 returns the total
__device__ __forceinline__ G1Jac block_sum_g1(G1Jac v) {
    __shared__ uint32_t lds[36][GT];
    const uint32_t t = threadIdx.x;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(&v);
#pragma unroll
    for (int l = 0; l < 36; ++l) lds[l][t] = src[l];
    __syncthreads();
    for (uint32_t s = GT / 2; s > 0; s >>= 1) {
        if (t < s) {
            G1Jac x, y;
            uint32_t* px = reinterpret_cast<uint32_t*>(&x);
            uint32_t* py = reinterpret_cast<uint32_t*>(&y);
#pragma unroll
            for (int l = 0; l < 36; ++l) { px[l] = lds[l][t]; py[l] = lds[l][t + s]; }
            x = g1_add(x, y);
#pragma unroll
            for (int l = 0; l < 36; ++l) lds[l][t] = px[l];
        }
        __syncthreads();
    }
    G1Jac r;
    uint32_t* pr = reinterpret_cast<uint32_t*>(&r);
#pragma unroll
    for (int l = 0; l < 36; ++l) pr[l] = lds[l][0];
    __syncthreads();
    return r;
}
// rows of length ncol: out[row] = sum_j in[row*ncol + j]; gridDim.y splits a row into segments
__global__ void __launch_bounds__(GT) k_g1_rowsum(G1Jac* __restrict__ out, const G1Jac* __restrict__ in, size_t ncol, uint32_t nseg) {
    const size_t row = blockIdx.x;
    const uint32_t seg = blockIdx.y;
    const size_t per = (ncol + nseg - 1) / nseg;
    const size_t j0 = seg * per, j1 = (j0 + per < ncol) ? j0 + per : ncol;
    G1Jac acc = g1_infinity();
    for (size_t j = j0 + threadIdx.x; j < j1; j += GT) acc = g1_add(acc, in[row * ncol + j]);
    acc = block_sum_g1(acc);
    if (threadIdx.x == 0) out[row * nseg + seg] = acc;
}

// ---- G1 multilinear fold step (G1_me_step, g1-tensor.cu:486-498); x is already "unmont"-ed ----------------
__global__ void __launch_bounds__(GT) k_g1_me_step(G1Jac* __restrict__ out, const G1Jac* __restrict__ in, const Fr x, size_t in_size, size_t out_size) {
    const size_t g = (size_t)blockIdx.x * GT + threadIdx.x;
    if (g >= out_size) return;
    const size_t g0 = 2 * g, g1 = 2 * g + 1;
    G1Jac r;
    if (g1 < in_size) r = g1_add(in[g0], g1_mul(g1_add(in[g1], g1_neg(in[g0])), x));
    else if (g0 < in_size) r = g1_add(in[g0], g1_neg(g1_mul(in[g0], x)));
    else r = g1_infinity();
    out[g] = r;
}

// ---- batch normalisation to z = 1 -------------------------------------------------------------------------
// Each lane owns CH consecutive points: prefix products of z, one Fermat inversion, back-substitution.
// Infinity (z == 0) is skipped in the product and written as all-zero limbs.
static constexpr int CH = 8;
template <bool AFFINE_OUT> __global__ void __launch_bounds__(GT) k_g1_normalize(void* outv, const G1Jac* in, size_t n) {
    const size_t base = ((size_t)blockIdx.x * GT + threadIdx.x) * CH;
    if (base >= n) return;
    Fp pre[CH];
    Fp run = big_one_mont<12>();
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        pre[c] = run;
        if (base + c < n) {
            const Fp z = in[base + c].z;
            if (!is_zero(z)) run = fp_mul(run, z);
        }
    }
    Fp inv = mont_inverse(run);
#pragma unroll
    for (int c = CH - 1; c >= 0; --c) {
        if (base + c >= n) continue;
        const G1Jac p = in[base + c];
        Fp ox = big_zero<12>(), oy = big_zero<12>(), oz = big_zero<12>();
        if (!is_zero(p.z)) {
            const Fp zi = fp_mul(inv, pre[c]);
            inv = fp_mul(inv, p.z);
            const Fp zi2 = fp_sqr(zi);
            ox = fp_mul(p.x, zi2);
            oy = fp_mul(fp_mul(p.y, zi2), zi);
            oz = big_one_mont<12>();
        }
        if (AFFINE_OUT) {
            G1Affine* out = reinterpret_cast<G1Affine*>(outv);
            out[base + c].x = ox; out[base + c].y = oy;
        } else {
            G1Jac* out = reinterpret_cast<G1Jac*>(outv);
            out[base + c].x = ox; out[base + c].y = oy; out[base + c].z = oz;
        }
    }
}

// the normalised points once more in the 29-bit-limb form that the bucket kernels add in (infinity stays all-zero)
__global__ void __launch_bounds__(256) k_g1aff_to_a29(A29* __restrict__ out, const G1Affine* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = a29_from_affine(in[i]);
}

// ---- fixed-base table for commit_int -------------------------------------------------------------------------
// table (Jacobian, before normalisation): tab[(w * ngen + j) * half + (d-1)] = d * 2^(c*w) * G_j, d = 1..half.
// Bases first, one lane per generator walking up the windows by c doublings each; then the multiples by doubling the
// filled part of every row, row[k + i] = row[i] + row[k - 1] for i < k, k = 1, 2, 4, ...: one launch per k with one lane
// per new entry, so every launch is dense whatever the row length (rows are as short as 4 entries when few tensor rows
// share the generators) and the chain of additions is log2(half) deep.
__global__ void __launch_bounds__(GT) k_msm_table_bases(G1Jac* __restrict__ tab, const G1Jac* __restrict__ gens, size_t ngen, uint32_t c, uint32_t nwin) {
    const size_t j = (size_t)blockIdx.x * GT + threadIdx.x;
    if (j >= ngen) return;
    const uint32_t half = 1u << (c - 1);
    G1Jac base = gens[j];
    for (uint32_t w = 0; w < nwin; ++w) {
        tab[((size_t)w * ngen + j) * half] = base;
        if (w + 1 < nwin) for (uint32_t k = 0; k < c; ++k) base = g1_double(base);
    }
}
__global__ void __launch_bounds__(GT) k_msm_table_fill(G1Jac* __restrict__ tab, size_t nrows, uint32_t logh, uint32_t logk) {
    const size_t t = (size_t)blockIdx.x * GT + threadIdx.x;
    if ((t >> logk) >= nrows) return;
    const uint32_t k = 1u << logk, i = (uint32_t)(t & (k - 1));
    G1Jac* row = tab + ((t >> logk) << logh);
    row[k + i] = g1_add(row[i], row[k - 1]);
}
// One workgroup per (row, segment): sum_j [s_j] G_j over the segment as mixed additions out of the
// affine table, in 29-bit limbs (the table is converted once per call).  Scalars are embedded int32 values
// (commit_int_dev_func, commitment.cu:31-42).
__global__ void __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_msm_rows(G1Jac* __restrict__ out, const A29* __restrict__ tab, const int32_t* __restrict__ scalars, size_t ngen, uint32_t c, uint32_t nwin, uint32_t nseg) {
    const size_t row = blockIdx.x;
    const uint32_t seg = blockIdx.y;
    const uint32_t half = 1u << (c - 1);
    const size_t per = (ngen + nseg - 1) / nseg;
    const size_t j0 = seg * per, j1 = (j0 + per < ngen) ? j0 + per : ngen;
    J29 acc29 = j29_infinity();
    for (size_t j = j0 + threadIdx.x; j < j1; j += GT) {
        const int32_t s = scalars[row * ngen + j];
        if (s == 0) continue;
        const bool negs = s < 0;
        uint64_t x = negs ? (uint64_t)(-(int64_t)s) : (uint64_t)s;
        for (uint32_t w = 0; w < nwin && x != 0; ++w) {
            int64_t d = (int64_t)(x & ((1u << c) - 1));
            x >>= c;
            if (d > (int64_t)half) { d -= (int64_t)(1u << c); x += 1; }
            if (d == 0) continue;
            const bool nd = (d < 0) != negs;
            const uint32_t mag = (uint32_t)(d < 0 ? -d : d);
            A29 p = tab[((size_t)w * ngen + j) * half + (mag - 1)];
            if (a29_is_inf(p)) continue;
            if (nd) p.y = fq29_neg(p.y);
            acc29 = j29_add_mixed(acc29, p);
        }
    }
    const G1Jac acc = block_sum_g1(j29_to_jac(acc29));
    if (threadIdx.x == 0) out[row * nseg + seg] = acc;
}
// out[i] = [s_i] B for one base point B: additions out of the table of B's multiples d * 2^(8w) B, d = 1..128, w = 0..32
// (signed 8-bit digits of the 256-bit integer s_i; window 32 only ever holds the last carry).  33 mixed additions at
// most instead of 255 doublings and ~128 additions.
static constexpr uint32_t FB_WIN = 33;
__global__ void __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_g1_fixed_base_mul(G1Jac* __restrict__ out, const A29* __restrict__ tab, const Fr* __restrict__ scalars, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= n) return;
    const Fr x = scalars[i];
    J29 acc29 = j29_infinity();
    uint32_t carry = 0;
    for (uint32_t w = 0; w < FB_WIN; ++w) {
        const uint32_t b = (w < 32 ? ((x.v[w >> 2] >> (8 * (w & 3))) & 255u) : 0u) + carry;
        carry = b > 128u ? 1u : 0u;
        const uint32_t mag = carry ? 256u - b : b;
        if (mag == 0) continue;
        A29 p = tab[w * 128u + (mag - 1)];
        if (a29_is_inf(p)) continue;
        if (carry) p.y = fq29_neg(p.y);
        acc29 = j29_add_mixed(acc29, p);
    }
    out[i] = j29_to_jac(acc29);
}
__global__ void __launch_bounds__(256) k_fr_to_i32_checked(int32_t* __restrict__ out, uint32_t* __restrict__ bad, uint32_t* __restrict__ maxabs, const Fr* __restrict__ in, size_t n) {
    __shared__ uint32_t wmax[4];
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint32_t a = 0;
    if (i < n) {
        const Fr x = in[i];
        // scalar_to_int semantics: values outside the int32 embedding collapse to what the reference reads
        const int32_t v = fr_to_i32(x);
        out[i] = v;
        const Fr back = fr_from_i64((int64_t)v);
        if (!equal(back, x)) atomicOr(bad, 1u);
        a = v < 0 ? (uint32_t)(-(int64_t)v) : (uint32_t)v;
    }
    // one atomic per workgroup: the largest magnitude of its 256 values
    for (int off = 32; off >= 1; off >>= 1) { const uint32_t o = (uint32_t)__shfl_xor((int)a, off, 64); a = o > a ? o : a; }
    if ((threadIdx.x & 63u) == 0) wmax[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t m = wmax[0];
        for (int k = 1; k < 4; ++k) m = wmax[k] > m ? wmax[k] : m;
        if (m) atomicMax(maxabs, m);
    }
}

// ---- opening (Commitment::me_open, commitment.cu:79-129) -------------------------------------------------------------
// A round of the opening halves the scalars s and the generators g with the challenge u,
//   s'_i = s_2i + u (s_2i+1 - s_2i),   g'_i = g_2i+1 + [u](g_2i - g_2i+1),
// and publishes T = sum [s_j] g_j, T0 = sum [s_2i] g_2i+1, T1 = sum [s_2i+1] g_2i.  The reference spends five
// 255-bit scalar multiplications per pair on this.  Here
//  * T0 and T1 (and T of the first round) are bucket multi-scalar multiplications over the affine-normalised
//    generators: 8-bit signed windows, one workgroup per (sum, window, segment), one bucket per lane;
//  * T of every later round follows from the previous round's three points, because <s', g'> expands to
//    u(1-u) T + (1-u)^2 T0 + u^2 T1;
//  * the one remaining scalar multiplication per pair, by the round's common challenge u, uses the curve
//    endomorphism (x, y) -> (beta x, y) = [lambda](x, y): u = k1 + k2 lambda with k1, k2 < 2^128 (r = lambda^2 +
//    lambda + 1, so this is one integer division on the host), then 128 doublings instead of 255.
// The endomorphism and the expansion of T hold for points of the order-r subgroup, which is where the
// generators live (Commitment::random draws multiples of the group generator, commitment.cu:9-20).
// All rounds are queued without a host round trip; the proof points come back in one copy, normalised to z = 1.
static constexpr int MW = 32;        // 8-bit signed windows over a 255-bit scalar
static constexpr int MT = 128;       // lanes of a bucket workgroup = buckets (digit magnitudes 1..128)
static constexpr int MSEG = 4096;    // elements per chunk (12-bit list entries)
static constexpr int MSL = 64;       // lanes of a bucket-accumulation workgroup (one wave): each takes two buckets of its chunk
static constexpr int MHEAVY = 256;   // a bucket above this many elements of a chunk is summed by the whole workgroup
struct MsmDesc { const int8_t* digits; const A29* base; uint32_t dstride, count, s_mul, s_off, b_mul, b_off, slot; };   // element i: recoded scalar i*s_mul+s_off of dstride, point base[i*b_mul+b_off]
static constexpr int OB_MAX = 8;           // openings of equal size that share their rounds' launches
static constexpr int OB_SUMS = 3 * OB_MAX;
template <int NMAX> struct MsmDescs { MsmDesc d[NMAX]; };
static constexpr int TAIL_N = 1024;        // generators at which the remaining rounds are computed in one batch (work grows with it, latency shrinks)
static constexpr int TAIL_LEVELS = 20;     // most rounds the batch takes
struct GlvK { uint32_t k1[4], k2[4]; };

__device__ __forceinline__ bool aff_is_inf(const G1Affine& p) { return is_zero(p.x) && is_zero(p.y); }   // normalised infinity: all-zero limbs
__device__ __forceinline__ G1Jac aff_to_jac(const G1Affine& p) {
    G1Jac r;
    if (aff_is_inf(p)) return g1_infinity();
    r.x = p.x; r.y = p.y; r.z = big_one_mont<12>();
    return r;
}
// beta (Montgomery form): the cube root of unity in Fp with (beta x, y) = [lambda](x, y), lambda = 0xac45a4010001a40200000000ffffffff
__device__ __forceinline__ Fp glv_beta() {
    Fp b;
    constexpr uint32_t t[12] = {2255614065u, 3439577572u, 533571026u, 1571496518u, 3548715925u, 1483752111u, 29019038u, 2394295998u, 2211467474u, 66682222u, 1415808833u, 418390117u};
#pragma unroll
    for (int i = 0; i < 12; ++i) b.v[i] = t[i];
    return b;
}
__device__ __forceinline__ Fp glv_beta2() {   // beta^2 = -1 - beta
    Fp b;
    constexpr uint32_t t[12] = {2039112936u, 821114395u, 2127452714u, 4088978859u, 3323295735u, 380160570u, 1962738331u, 3261739000u, 1617960046u, 909555558u, 605774176u, 85697707u};
#pragma unroll
    for (int i = 0; i < 12; ++i) b.v[i] = t[i];
    return b;
}
__device__ __forceinline__ Fp glv_minus2_over_beta_minus_1() {   // -2 / (beta - 1), Montgomery form
    Fp b;
    constexpr uint32_t t[12] = {72385493u, 4027593027u, 4077721914u, 4036542869u, 1636888181u, 235204061u, 17598343u, 35324347u, 360752738u, 1434563812u, 3508079257u, 43087383u};
#pragma unroll
    for (int i = 0; i < 12; ++i) b.v[i] = t[i];
    return b;
}
// joint sparse form of (k1, k2): position i holds (d1 + 1) | (d2 + 1) << 2 in 4 bits, d in {-1, 0, 1}; len <= 129
struct JsfK { uint32_t dig[17]; uint32_t len; };
// [k1]P + [k2]phi(P); every lane of a wave must carry the same k (the add pattern is uniform)
static __device__ __attribute__((noinline)) G1Jac g1_mul_glv(const G1Jac& P, const GlvK& k) {
    if (is_zero(P.z)) return P;
    G1Jac Q = P;
    Q.x = fp_mul(P.x, glv_beta());
    const G1Jac PQ = g1_add(P, Q);
    int top = -1;
    for (int i = 3; i >= 0 && top < 0; --i) {
        const uint32_t x = k.k1[i] | k.k2[i];
        if (x) top = i * 32 + 31 - __builtin_clz(x);
    }
    G1Jac out = g1_infinity();
    for (int i = top; i >= 0; --i) {
        out = g1_double(out);
        const uint32_t b = ((k.k1[i >> 5] >> (i & 31)) & 1u) | (((k.k2[i >> 5] >> (i & 31)) & 1u) << 1);
        if (b == 1) out = g1_add(out, P);
        else if (b == 2) out = g1_add(out, Q);
        else if (b == 3) out = g1_add(out, PQ);
    }
    return out;
}

// Signed 8-bit digits of the balanced representative of every scalar, written window-major: D[w*n + i] in [-128, 127]
// for w < MW, and D[MW*n + i] = 1 when the scalar was replaced by r - s (its point is then subtracted).  Taking the
// smaller of s and r - s gives small negative values (r - x, as weights are embedded) as few non-zero windows as
// small positive ones, instead of r's high bytes in every one of them.  A window byte above 127 becomes byte - 256
// and carries one into the next window; the top window of a value below 2^254 cannot overflow.
struct RecodeBatch { int8_t* D[OB_MAX]; const Fr* S[OB_MAX]; };      // blockIdx.y names the pair
// the digits of scalar i of n (standard form)
__device__ __forceinline__ void msm_recode_store(int8_t* __restrict__ D, size_t n, size_t i, const Fr& sv) {
    Fr ng;
    uint32_t br = 0;
#pragma unroll
    for (int l = 0; l < 8; ++l) ng.v[l] = subb32(FrK::P(l), sv.v[l], br);
    uint32_t lt = 0;    // borrow of (r - s) - s: r - s is the smaller one
#pragma unroll
    for (int l = 0; l < 8; ++l) (void)subb32(ng.v[l], sv.v[l], lt);
    const bool flip = lt != 0;
    uint32_t carry = 0;
#pragma unroll
    for (int l = 0; l < 8; ++l) {
        const uint32_t word = flip ? ng.v[l] : sv.v[l];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t raw = ((word >> (8 * q)) & 0xFFu) + carry;
            carry = raw > 127u ? 1u : 0u;
            D[(size_t)(4 * l + q) * n + i] = (int8_t)(raw > 127u ? (int)raw - 256 : (int)raw);
        }
    }
    D[(size_t)MW * n + i] = flip ? 1 : 0;
}
__global__ void __launch_bounds__(256) k_msm_recode(const RecodeBatch rb, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    msm_recode_store(rb.D[blockIdx.y], n, i, rb.S[blockIdx.y][i]);
}

// sum over the NT lanes of a workgroup through the LDS pool (36 x NT words); every lane returns the total
template <int NT = MT> __device__ __forceinline__ G1Jac msm_block_sum(uint32_t* pool, const G1Jac& v, uint32_t t) {
    __syncthreads();
    {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(&v);
#pragma unroll
        for (int l = 0; l < 36; ++l) pool[l * NT + t] = src[l];
    }
    __syncthreads();
    for (uint32_t sd = NT / 2; sd > 0; sd >>= 1) {
        if (t < sd) {
            G1Jac x, y;
            uint32_t* px = reinterpret_cast<uint32_t*>(&x);
            uint32_t* py = reinterpret_cast<uint32_t*>(&y);
#pragma unroll
            for (int l = 0; l < 36; ++l) { px[l] = pool[l * NT + t]; py[l] = pool[l * NT + t + sd]; }
            x = g1_add(x, y);
#pragma unroll
            for (int l = 0; l < 36; ++l) pool[l * NT + t] = px[l];
        }
        __syncthreads();
    }
    G1Jac tot;
    uint32_t* pr = reinterpret_cast<uint32_t*>(&tot);
#pragma unroll
    for (int l = 0; l < 36; ++l) pr[l] = pool[l * NT];
    __syncthreads();
    return tot;
}

// One segment's share of sum over elements of digit_w(s) * base: the segment's MT raw buckets,
// partial[((sum * MW + w) * nseg + seg) * MT + b] for bucket magnitude b + 1 (k_msm_bucket_fold / k_msm_point reduce them).
// One wave per workgroup.  Per chunk of MSEG elements:
//  1. the bucket sizes are counted (one LDS atomic per element) and the elements are sorted by bucket into one list in
//     LDS (counting sort: 12-bit position in the chunk + sign);
//  2. the buckets are ranked by size and lane j takes the j-th largest and the j-th smallest: list lengths of uniform
//     digits are Poisson(32), the largest of 64 is ~47, while the 64 pair sums all lie within a few elements of 64 -- the
//     lanes walk their two lists as one sequence of mixed additions, in lockstep, and 96 % of the lane-steps add a point
//     (67 % with one bucket per lane);
//  3. a bucket with more than MHEAVY elements (scalars that share a digit: equal values, a common high byte) is left out
//     of the lists and summed by all lanes together, each over its own share of the chunk.
template <int NMAX>
__global__ void __launch_bounds__(MSL) __attribute__((amdgpu_waves_per_eu(2, 2))) k_msm_seg(G1Jac* __restrict__ partial, const MsmDescs<NMAX> descs, const MsmDesc* __restrict__ ddescs, uint32_t nseg, uint32_t chunks_per_seg) {
    __shared__ uint32_t cnt[MT], off[MT], cursor[MT];
    __shared__ uint8_t order[MT];
    __shared__ uint32_t pool[36 * MSL];            // the sorted list (u16 x MSEG), then the 36 x MSL point tree of the heavy buckets
    static_assert(36 * MSL * 4 >= MSEG * 2, "pool too small for the list");
    static_assert(MSEG <= 4096, "12-bit list entries");
    uint16_t* list = reinterpret_cast<uint16_t*>(pool);
    const MsmDesc d = ddescs ? ddescs[blockIdx.z] : descs.d[blockIdx.z];      // many sums: the descriptors lie in device memory
    const A29* __restrict__ A = d.base;
    const uint32_t w = blockIdx.y, seg = blockIdx.x, t = threadIdx.x, zz = blockIdx.z;
    const int8_t* __restrict__ Dw = d.digits + (size_t)w * d.dstride;
    const int8_t* __restrict__ Df = d.digits + (size_t)MW * d.dstride;
    G1Jac* __restrict__ out = partial + (((size_t)zz * MW + w) * nseg + seg) * MT;
    bool first = true;                                  // nothing written to `out` yet (the same for every lane)
    for (uint32_t ch = 0; ch < chunks_per_seg; ++ch) {
        const uint32_t e0 = (seg * chunks_per_seg + ch) * MSEG;
        if (e0 >= d.count) break;
        const uint32_t e1 = (e0 + MSEG < d.count) ? e0 + MSEG : d.count;
        cnt[t] = 0; cnt[t + MSL] = 0;
        __syncthreads();
        for (uint32_t e = e0 + t; e < e1; e += MSL) {
            const int dg = Dw[(size_t)e * d.s_mul + d.s_off];
            if (dg != 0) atomicAdd(&cnt[(dg < 0 ? -dg : dg) - 1], 1u);
        }
        __syncthreads();
        if (t == 0) {
            uint32_t run = 0;
            for (uint32_t b = 0; b < (uint32_t)MT; ++b) {
                off[b] = run; cursor[b] = run;
                run += cnt[b] > (uint32_t)MHEAVY ? 0u : cnt[b];
            }
        }
        // rank of a bucket by list length (heavy buckets have none), ties by index: a permutation
        for (uint32_t b = t; b < (uint32_t)MT; b += MSL) {
            const uint32_t cb = cnt[b] > (uint32_t)MHEAVY ? 0u : cnt[b];
            uint32_t r = 0;
            for (uint32_t o = 0; o < (uint32_t)MT; ++o) {
                const uint32_t co = cnt[o] > (uint32_t)MHEAVY ? 0u : cnt[o];
                r += (co > cb || (co == cb && o < b)) ? 1u : 0u;
            }
            order[r] = (uint8_t)b;
        }
        __syncthreads();
        for (uint32_t e = e0 + t; e < e1; e += MSL) {
            const size_t si = (size_t)e * d.s_mul + d.s_off;
            const int dg = Dw[si];
            if (dg == 0) continue;
            const uint32_t mag = (uint32_t)(dg < 0 ? -dg : dg);
            if (cnt[mag - 1] > (uint32_t)MHEAVY) continue;
            const uint32_t pos = atomicAdd(&cursor[mag - 1], 1u);
            list[pos] = (uint16_t)((e - e0) | (((dg < 0) != (Df[si] != 0)) ? 0x8000u : 0u));
        }
        __syncthreads();
        {
            const uint32_t bA = order[t], bB = order[MT - 1 - t];
            const uint32_t lenA = cnt[bA] > (uint32_t)MHEAVY ? 0u : cnt[bA], lenB = cnt[bB] > (uint32_t)MHEAVY ? 0u : cnt[bB];
            const uint32_t total = lenA + lenB;
            uint32_t pos = off[bA];
            J29 acc29 = j29_infinity();
            for (uint32_t i = 0;; ++i) {
                if (i == lenA) {
                    // the end of the first list: its bucket goes out (added to what earlier chunks of this segment left there)
                    G1Jac v = j29_to_jac(acc29);
                    if (!first) v = g1_add(out[bA], v);
                    out[bA] = v;
                    acc29 = j29_infinity();
                    pos = off[bB];
                }
                if (i >= total) break;
                const uint32_t en = list[pos++];
                A29 pt = A[(size_t)(e0 + (en & 0x7FFFu)) * d.b_mul + d.b_off];
                if (a29_is_inf(pt)) continue;
                if (en & 0x8000u) pt.y = fq29_neg(pt.y);
                acc29 = j29_add_mixed(acc29, pt);
            }
            G1Jac v = j29_to_jac(acc29);
            if (!first) v = g1_add(out[bB], v);
            out[bB] = v;
        }
        __threadfence_block();
        __syncthreads();
        for (uint32_t b = 0; b < (uint32_t)MT; ++b) {
            if (cnt[b] <= (uint32_t)MHEAVY) continue;          // the same for every lane
            J29 h29 = j29_infinity();
            for (uint32_t e = e0 + t; e < e1; e += MSL) {
                const size_t si = (size_t)e * d.s_mul + d.s_off;
                const int dg = Dw[si];
                if ((uint32_t)(dg < 0 ? -dg : dg) != b + 1) continue;
                A29 pt = A[(size_t)e * d.b_mul + d.b_off];
                if (a29_is_inf(pt)) continue;
                if ((dg < 0) != (Df[si] != 0)) pt.y = fq29_neg(pt.y);
                h29 = j29_add_mixed(h29, pt);
            }
            const G1Jac h = msm_block_sum<MSL>(pool, j29_to_jac(h29), t);
            if (t == 0) out[b] = g1_add(out[b], h);            // its list was empty: the slot holds what earlier chunks left (or infinity)
        }
        __threadfence_block();
        __syncthreads();
        first = false;
    }
    if (first) {                                       // a segment past the end of this sum: empty buckets
        out[t] = g1_infinity();
        out[t + MSL] = g1_infinity();
    }
}
// raw buckets of up to 8 consecutive segments summed: out[(row * gridDim.y + group) * MT + t], row = sum * MW + w
__global__ void __launch_bounds__(MT) k_msm_bucket_fold(G1Jac* __restrict__ out, const G1Jac* __restrict__ buckets, uint32_t nseg) {
    const uint32_t t = threadIdx.x, row = blockIdx.x, grp = blockIdx.y;
    const uint32_t s0 = grp * 8, s1 = (s0 + 8 < nseg) ? s0 + 8 : nseg;
    const G1Jac* b = buckets + (size_t)row * nseg * MT;
    G1Jac acc = b[(size_t)s0 * MT + t];
    for (uint32_t sg = s0 + 1; sg < s1; ++sg) acc = g1_add(acc, b[(size_t)sg * MT + t]);
    out[((size_t)row * gridDim.y + grp) * MT + t] = acc;
}
// The whole sum from the raw buckets of all its windows, one workgroup per sum: lane t first combines bucket t+1 over the
// windows, sum_w 2^(8w) B[w][t+1] (one Horner walk of 248 doublings, the segments of a window added on the way), and only
// then weights it by t+1 -- one weighting and one lane sum per sum instead of one per window, and no Horner pass of a
// single lane over window sums afterwards.  Raw buckets: buckets[((z MW + w) nseg + seg) MT + t].  wsum != nullptr: the point
// goes where k_open_horner expects the window sums of sum z, wsum[(z / n_per) item_stride + (z % n_per) MW + w] (the sums of one
// opening lie together, the openings of a batch item_stride apart): the point as window 0, infinity above; else into
// pts[descs[z].slot].
// list != nullptr: sum z is list[z] -- its raw buckets, their segment count and where its window sums go (the sums of
// several rounds of a job in one launch, behind the last round's bucket accumulation).
struct PointDesc { const G1Jac* buckets; G1Jac* W; uint32_t nseg, pad; };
__global__ void __launch_bounds__(MT) k_msm_point(G1Jac* __restrict__ wsum, G1Jac* __restrict__ pts, const MsmDesc* __restrict__ descs, const G1Jac* __restrict__ buckets,
                                                  uint32_t nseg, uint32_t n_per, uint32_t item_stride, const PointDesc* __restrict__ list) {
    __shared__ uint32_t pool[36 * MT];
    const uint32_t t = threadIdx.x, z = blockIdx.x;
    if (list) { buckets = list[z].buckets; nseg = list[z].nseg; }
    const size_t zb = list ? 0 : z;
    // The walk is one lane's chain of 248 doublings: it runs in 29-bit limbs (two thirds of the instructions of the 32-bit
    // formulas, and the point stays in registers instead of travelling through private memory at every call).
    J29 r = j29_infinity();
    for (int w = MW - 1; w >= 0; --w) {
        if (w != MW - 1)
            for (int k = 0; k < 8; ++k) r = j29_double(r);
        const G1Jac* b = buckets + (zb * MW + (uint32_t)w) * nseg * MT;
        for (uint32_t sg = 0; sg < nseg; ++sg) {
            const G1Jac pt = b[(size_t)sg * MT + t];
            if (!is_zero(pt.z)) r = j29_add(r, j29_from_jac(pt));
        }
    }
    J29 q29 = j29_infinity();
    for (int bit = 7; bit >= 0; --bit) {
        q29 = j29_double(q29);
        if (((t + 1) >> bit) & 1u) q29 = j29_add(q29, r);
    }
    const G1Jac q = j29_to_jac(q29);
    const G1Jac tot = msm_block_sum(pool, q, t);
    if (wsum || list) {
        G1Jac* __restrict__ W = list ? list[z].W : wsum + (size_t)(z / n_per) * item_stride + (size_t)(z % n_per) * MW;
        if (t == 0) W[0] = tot;
        else if (t < (uint32_t)MW) W[t] = g1_infinity();
    } else if (t == 0) pts[descs[z].slot] = tot;
}

// ---- the single points of the halving rounds, once per opening ---------------------------------------------------------
// None of this feeds a fold, so nothing of it sits between two rounds: the rounds only leave their window sums behind
// (W[(3 * round + j) * MW + w], j = 0, 1, 2 for T, T0, T1), and after the last round
//  k_open_horner assembles every sum from its windows, sum_w 2^(8w) W[w], one lane per sum, all sums side by side;
//  k_open_chain  computes T of every round r >= 1 (the reference sums s_i g_i over the folded vectors, commitment.cu:103): unrolling
//                T_r = u(1-u) T_(r-1) + (1-u)^2 T0_(r-1) + u^2 T1_(r-1)   (u = the challenge of round r-1)
//                down to round 0 makes T_r a combination of T_0 and the T0, T1 of the rounds before r with coefficients
//                that are products of the challenges -- all rounds at once, one lane per term.
// blockIdx.y: the opening of a batch (its points npts apart, its window sums wstride apart)
__global__ void __launch_bounds__(GT) k_open_horner(G1Jac* __restrict__ pts0, const G1Jac* __restrict__ Wall0, uint32_t halving_rounds, uint32_t npts, uint32_t wstride) {
    if (threadIdx.x != 0) return;
    G1Jac* __restrict__ pts = pts0 + (size_t)blockIdx.y * npts;
    const G1Jac* __restrict__ Wall = Wall0 + (size_t)blockIdx.y * wstride;
    const uint32_t x = blockIdx.x, round = x / 3, j = x % 3;
    if (round >= halving_rounds || (round > 0 && j == 0)) return;
    const G1Jac* W = Wall + (size_t)x * MW;
    G1Jac r = W[MW - 1];
    for (int w = MW - 2; w >= 0; --w) {
        for (int k = 0; k < 8; ++k) r = g1_double(r);
        r = g1_add(r, W[w]);
    }
    pts[x] = r;
}
// k = k1 + k2 * lambda, 0 <= k1 < lambda (r = lambda^2 + lambda + 1, so k2 <= lambda + 1): one long division, as glv_split on the host
__device__ __forceinline__ GlvK glv_split_device(const Fr& k) {
    const uint64_t lam_hi = 0xac45a4010001a402ull, lam_lo = 0x00000000ffffffffull;
    uint64_t rh = 0, rl = 0, qh = 0, ql = 0;
    for (int i = 255; i >= 0; --i) {
        const bool top = (rh >> 63) != 0;
        rh = (rh << 1) | (rl >> 63);
        rl = (rl << 1) | ((k.v[i >> 5] >> (i & 31)) & 1u);
        qh = (qh << 1) | (ql >> 63);
        ql <<= 1;
        if (top || rh > lam_hi || (rh == lam_hi && rl >= lam_lo)) {
            const uint64_t nl = rl - lam_lo;
            rh = rh - lam_hi - (rl < lam_lo ? 1u : 0u);
            rl = nl;
            ql |= 1u;
        }
    }
    GlvK o;
    o.k1[0] = (uint32_t)rl; o.k1[1] = (uint32_t)(rl >> 32); o.k1[2] = (uint32_t)rh; o.k1[3] = (uint32_t)(rh >> 32);
    o.k2[0] = (uint32_t)ql; o.k2[1] = (uint32_t)(ql >> 32); o.k2[2] = (uint32_t)qh; o.k2[3] = (uint32_t)(qh >> 32);
    return o;
}
// [k1]P + [k2]phi(P) with a k of the lane's own: one doubling and at most one addition per bit, whatever the other lanes hold
static __device__ __attribute__((noinline)) G1Jac g1_mul_glv_lane(const G1Jac& P, const GlvK& k) {
    G1Jac Q = P;
    Q.x = fp_mul(P.x, glv_beta());
    const G1Jac PQ = g1_add(P, Q);
    G1Jac out = g1_infinity();
    for (int i = 127; i >= 0; --i) {
        out = g1_double(out);
        const uint32_t b = ((k.k1[i >> 5] >> (i & 31)) & 1u) | (((k.k2[i >> 5] >> (i & 31)) & 1u) << 1);
        if (b) {
            const G1Jac t = b == 1 ? P : (b == 2 ? Q : PQ);
            out = g1_add(out, t);
        }
    }
    return out;
}
// the same walk in 29-bit limbs.  P stays in registers; beta x (the abscissa of phi(P)) and P + phi(P) wait in LDS, word-
// interleaved over the workgroup's NT lanes (tab: 57 x NT words), so the walk fits the register file without spilling.
template <int NT> static __device__ J29 j29_mul_glv_lane(const J29& P, const GlvK& k, int32_t (*tab)[NT]) {
    const uint32_t t = threadIdx.x;
    {
        J29 Q = P;
        Q.x = fq29_mul(P.x, fq29_from_fp(glv_beta()));
        const J29 PQ = j29_add(P, Q);
#pragma unroll
        for (int l = 0; l < 14; ++l) { tab[l][t] = Q.x.l[l]; tab[14 + l][t] = PQ.x.l[l]; tab[28 + l][t] = PQ.y.l[l]; tab[42 + l][t] = PQ.z.l[l]; }
        tab[56][t] = (int32_t)PQ.inf;
    }
    J29 out = j29_infinity();
    for (int i = 127; i >= 0; --i) {
        out = j29_double(out);
        const uint32_t b = ((k.k1[i >> 5] >> (i & 31)) & 1u) | (((k.k2[i >> 5] >> (i & 31)) & 1u) << 1);
        if (b) {
            J29 a = P;
            if (b == 2) {
#pragma unroll
                for (int l = 0; l < 14; ++l) a.x.l[l] = tab[l][t];
            } else if (b == 3) {
#pragma unroll
                for (int l = 0; l < 14; ++l) { a.x.l[l] = tab[14 + l][t]; a.y.l[l] = tab[28 + l][t]; a.z.l[l] = tab[42 + l][t]; }
                a.inf = (uint32_t)tab[56][t];
            }
            out = j29_add(out, a);
        }
    }
    return out;
}
// grid: halving_rounds - 1 workgroups; workgroup x computes T of round x + 1 into pts[3 * (x + 1)].  Needs T_0 and all T0, T1.
// U: the openings' challenges in Montgomery form, opening y's at U + y * ustride
__global__ void __launch_bounds__(GT) k_open_chain(G1Jac* __restrict__ pts0, const Fr* __restrict__ U, uint32_t halving_rounds, uint32_t npts, uint32_t ustride) {
    __shared__ uint32_t pool[36 * GT];
    __shared__ int32_t walk_tab[57][GT];
    G1Jac* __restrict__ pts = pts0 + (size_t)blockIdx.y * npts;
    const Fr* __restrict__ usu = U + (size_t)blockIdx.y * ustride;
    const uint32_t r = blockIdx.x + 1, t = threadIdx.x;
    const Fr one = big_one_mont<8>();
    G1Jac acc = g1_infinity();
    if (r < halving_rounds) {
        for (uint32_t i = t; i < 2 * r + 1; i += GT) {
            // term i: i == 0 -> T_0 with prod_{j<r} a_j;  i = 1 + 2k + s -> (s ? T1_k : T0_k) with (s ? u_k^2 : (1-u_k)^2) prod_{k<j<r} a_j,  a_j = u_j (1 - u_j)
            const uint32_t k = i == 0 ? 0u : (i - 1) / 2, s1 = i == 0 ? 0u : (i - 1) & 1u;
            Fr c = one;
            for (uint32_t j = (i == 0 ? 0u : k + 1); j < r; ++j) c = mont_mul(c, mont_mul(usu[j], sub(one, usu[j])));
            if (i != 0) {
                const Fr f = s1 ? usu[k] : sub(one, usu[k]);
                c = mont_mul(c, mont_mul(f, f));
            }
            const G1Jac P = pts[i == 0 ? 0u : 3 * k + 1 + s1];
            if (!is_zero(P.z)) acc = g1_add(acc, j29_to_jac(j29_mul_glv_lane<GT>(j29_from_jac(P), glv_split_device(from_mont(c)), walk_tab)));
        }
    }
    // sum over the lanes
    __syncthreads();
    {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(&acc);
#pragma unroll
        for (int l = 0; l < 36; ++l) pool[l * GT + t] = src[l];
    }
    __syncthreads();
    for (uint32_t sd = GT / 2; sd > 0; sd >>= 1) {
        if (t < sd) {
            G1Jac x, y;
            uint32_t* px = reinterpret_cast<uint32_t*>(&x);
            uint32_t* py = reinterpret_cast<uint32_t*>(&y);
#pragma unroll
            for (int l = 0; l < 36; ++l) { px[l] = pool[l * GT + t]; py[l] = pool[l * GT + t + sd]; }
            x = g1_add(x, y);
#pragma unroll
            for (int l = 0; l < 36; ++l) pool[l * GT + t] = px[l];
        }
        __syncthreads();
    }
    if (t == 0 && r < halving_rounds) {
        G1Jac tot;
        uint32_t* pr = reinterpret_cast<uint32_t*>(&tot);
#pragma unroll
        for (int l = 0; l < 36; ++l) pr[l] = pool[l * GT];
        pts[3 * r] = tot;
    }
}
// Sums of an opening's first rounds from commitments of the opened tensor's rows.  The opened vector is the row fold of a
// tensor W, s = sum_r e_r W[r] with e_r = prod_j (bit_j(r) ? v_j : 1 - v_j) over the row challenges v, so every sum of the
// form  sum_j s_(L j + x) g_(L j + y)  equals  sum_r e_r X[r]  with  X[r] = sum_j W[r][L j + x] g_(L j + y),  a point that
// depends on the tensor and the generators alone and can be made in advance (a commitment of a strided part of the row
// under a strided part of the generators).  T0 and T1 of round q are combinations of 4^q such sums each: with u_0 .. u_(q-1)
// the challenges of the rounds before,
//   s^(q)_m = sum_{a < 2^q} s_(2^q m + a) prod_k (bit_k(a) ? u_k : 1 - u_k),   g^(q)_m = sum_{b < 2^q} g_(2^q m + b) prod_k (bit_k(b) ? 1 - u_k : u_k),
//   T0_q = sum_j s^(q)_(2j) g^(q)_(2j+1) = sum_{a,b} c(a,b) sum_j s_(2^(q+1) j + a) g_(2^(q+1) j + 2^q + b),   T1_q likewise with the halves exchanged,
// and T of round 0 is the same combination of the row commitments themselves.  `pts`: [pattern][row] points, pattern 0 the row
// commitments, then for q = 0 .. cross_rounds - 1 the 4^q patterns (a 2^q + b) of T0_q followed by those of T1_q.
// Target t of an opening: 0 = T of round 0, 1 + 2q + side = T0_q / T1_q.  The results go where k_open_horner reads the window
// sums of those points: the point in window 0, infinity above.  They equal the sums over all generators exactly when `pts`
// are such commitments of the opened tensor -- what the caller states by passing them.
__host__ __device__ __forceinline__ void cross_target(uint32_t t, uint32_t& q, uint32_t& first_pattern, uint32_t& npat, uint32_t& slot) {
    if (t == 0) { q = 0; first_pattern = 0; npat = 1; slot = 0; return; }
    q = (t - 1) >> 1;
    const uint32_t side = (t - 1) & 1u, four_q = 1u << (2 * q);
    npat = four_q;
    first_pattern = 1 + 2 * (four_q - 1) / 3 + side * four_q;
    slot = (3 * q + 1 + side) * (uint32_t)MW;
}
// These sums are bucket multi-scalar multiplications.  Term g = pattern * nrows + row of an opening, in the order `pts`
// lays the points out, has the coefficient eq(u_rows, row) * c(pattern) -- c = 1 for the row commitments, the product of the
// earlier rounds' challenges for a cross pattern -- and a target is the sum over a contiguous range of terms: one bucket sum
// per target over the normalised points, with the digits of all terms written once, as k_msm_recode writes them
// (D: (MW + 1) x terms bytes).  A term costs 32 mixed additions (a scalar multiplication of its own would cost a 129-step walk).
struct CrossDigitItem { int8_t* D; const Fr* u_rows; const Fr* u; uint32_t nrows, k_rows; };
struct CrossDigitBatch { CrossDigitItem it[OB_MAX]; };
// grid (ceil(most terms / 256), openings)
__global__ void __launch_bounds__(256) k_open_cross_digits(const CrossDigitBatch cb, uint32_t npatterns) {
    const CrossDigitItem& it = cb.it[blockIdx.y];
    const size_t terms = (size_t)npatterns * it.nrows, i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= terms) return;
    const uint32_t p = (uint32_t)(i / it.nrows), row = (uint32_t)(i - (size_t)p * it.nrows);
    const Fr one = big_one_mont<8>();
    Fr coef = one;
    for (uint32_t j = 0; j < it.k_rows; ++j) coef = mont_mul(coef, ((row >> j) & 1u) ? it.u_rows[j] : sub(one, it.u_rows[j]));
    if (p != 0) {
        uint32_t q = 0, first = 1;                      // the patterns of round q: T0's 4^q, then T1's
        while (p >= first + (2u << (2 * q))) { first += 2u << (2 * q); ++q; }
        const uint32_t pl = (p - first) & ((1u << (2 * q)) - 1u), a = pl >> q, b = pl & ((1u << q) - 1u);
        for (uint32_t k = 0; k < q; ++k) {
            const Fr uk = it.u[k], nk = sub(one, uk);
            coef = mont_mul(coef, mont_mul(((a >> k) & 1u) ? uk : nk, ((b >> k) & 1u) ? nk : uk));
        }
    }
    msm_recode_store(it.D, terms, i, from_mont(coef));
}
// ---- the fold on 29-bit-limb affine points ----------------------------------------------------------------------------------
// The rounds of an opening keep the generators in ONE form: affine, 29-bit limbs (A29; all-zero limbs = infinity), canonical
// limbs.  The bucket sums add out of it, the fold reads it and writes the next round's generators in it -- no
// normalisation or conversion pass between two rounds.
// 1 / v for every lane of a 64-lane workgroup with one field inversion (product tree in LDS; the root goes through the
// 32-bit form, where the binary inverse lives).  v must not be 0 mod p (lanes with nothing to invert pass one).
// lds: 14 x 128 words.
__device__ __forceinline__ Fq29 block_inv64_29(const Fq29& v, int32_t (*lds)[2 * GT]) {
    const uint32_t t = threadIdx.x;
    auto put = [&](const Fq29& x, uint32_t i) {
#pragma unroll
        for (int l = 0; l < 14; ++l) lds[l][i] = x.l[l];
    };
    auto get = [&](uint32_t i) {
        Fq29 x;
#pragma unroll
        for (int l = 0; l < 14; ++l) x.l[l] = lds[l][i];
        return x;
    };
    __syncthreads();
    put(v, t);
    __syncthreads();
    uint32_t off = 0;
    for (uint32_t cnt = GT / 2; cnt >= 1; cnt >>= 1) {
        const uint32_t noff = off + 2 * cnt;
        if (t < cnt) put(fq29_mul(get(off + 2 * t), get(off + 2 * t + 1)), noff + t);
        __syncthreads();
        off = noff;
    }
    {
        const Fq29 root_inv = fq29_from_fp(mont_inverse(fq29_to_fp(get(off))));      // every lane the same value: no divergence
        __syncthreads();
        if (t == 0) put(root_inv, off);
        __syncthreads();
    }
    for (uint32_t cnt = 1; cnt < (uint32_t)GT; cnt <<= 1) {
        const uint32_t coff = off - 2 * cnt;
        Fq29 c = fq29_one();
        if (t < 2 * cnt) c = fq29_mul(get(off + (t >> 1)), get(coff + (t ^ 1u)));
        __syncthreads();
        if (t < 2 * cnt) put(c, coff + t);
        __syncthreads();
        off = coff;
    }
    const Fq29 r = get(t);
    __syncthreads();
    return r;
}
struct FoldItem { Fr* ns; A29* ng; const Fr* s; const A29* g; uint32_t* special; Fr u_mont; JsfK jsf; };
struct FoldBatch { FoldItem it[OB_MAX]; };          // blockIdx.y names the opening; all of one size
// Pair g of the round: s' and g' = a1 + [u](a0 - a1), all in 29-bit limbs.  The scalar multiplication walks the joint
// sparse form of the split challenge over the all-affine table {D, phi(D), D + phi(D), D - phi(D)}, D = a0 - a1, and the
// result is brought back to affine form in the kernel (a third inversion batched over the 64 lanes).  Pairs whose inputs
// are special (a0 at infinity, equal abscissae, an abscissa of zero) are not computed here: their indices go to
// `special` ([0] = count, then the indices) and k_open_fold_special takes them.
__global__ void __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_open_fold29(const FoldBatch fb, size_t old_size, size_t new_size) {
    Fr* __restrict__ new_scalars = fb.it[blockIdx.y].ns;
    A29* __restrict__ new_gens = fb.it[blockIdx.y].ng;
    const Fr* __restrict__ scalars = fb.it[blockIdx.y].s;
    const A29* __restrict__ A = fb.it[blockIdx.y].g;
    uint32_t* __restrict__ special = fb.it[blockIdx.y].special;
    const Fr u_mont = fb.it[blockIdx.y].u_mont;
    const JsfK& jsf = fb.it[blockIdx.y].jsf;
    __shared__ int32_t fold_lds[4 * 14 * GT];
    static_assert(4 * 14 * GT >= 14 * 2 * GT, "the inversion buffer shares the table's space");
    int32_t (*inv_lds)[2 * GT] = reinterpret_cast<int32_t (*)[2 * GT]>(fold_lds);
    int32_t (*tab)[14][GT] = reinterpret_cast<int32_t (*)[14][GT]>(fold_lds);
    const size_t g = (size_t)blockIdx.x * GT + threadIdx.x;
    const bool live = g < new_size;
    const size_t g0 = 2 * g, g1 = 2 * g + 1;
    const bool has1 = live && g1 < old_size;
    A29 a0, a1;
    a0.x = a0.y = a1.x = a1.y = fq29_zero();
    if (live) a0 = A[g0];
    if (has1) a1 = A[g1];
    if (live) {
        if (has1) new_scalars[g] = add(scalars[g0], mont_mul(u_mont, sub(scalars[g1], scalars[g0])));
        else new_scalars[g] = sub(scalars[g0], mont_mul(u_mont, scalars[g0]));
    }
    const bool inf0 = a29_is_inf(a0), inf1 = !has1 || a29_is_inf(a1);
    const Fq29 one29 = fq29_one();
    bool general = live && inf0;
    Fq29 den = one29;
    if (live && !general && !inf1) {
        den = fq29_sub(a0.x, a1.x);
        if (fq29_is_zero_mod_p(den)) { general = true; den = one29; }
    }
    const bool need_sub = live && !general && !inf1;          // D = a0 - a1 needs 1 / (x0 - x1)
    Fq29 inv = block_inv64_29(den, inv_lds);
    Fq29 xD = a0.x, yD = a0.y;
    if (need_sub) {
        const Fq29 lam = fq29_mul(fq29_add(a0.y, a1.y), inv);          // -a1 = (x1, -y1)
        const Fq29 x3 = fq29_sub(fq29_sub(fq29_sqr(lam), a0.x), a1.x);
        yD = fq29_mul(fq29_sub(fq29_mul(lam, fq29_sub(a0.x, x3)), a0.y), one29);      // the products by one bring the sums back into (-eps, p + eps)
        xD = fq29_mul(x3, one29);
    }
    if (live && !general && fq29_is_zero_mod_p(xD)) general = true;       // x = 0: not in the subgroup; the table below would divide by it
    const bool fast = live && !general;
    inv = block_inv64_29(fast ? xD : one29, inv_lds);
    J29 w = j29_infinity();
    if (fast) {
        {
            const Fq29 xQ = fq29_mul(xD, fq29_from_fp(glv_beta())), xPQ = fq29_mul(xD, fq29_from_fp(glv_beta2()));
            const Fq29 lam = fq29_mul(fq29_mul(fq29_from_fp(glv_minus2_over_beta_minus_1()), yD), inv);   // slope of D + (beta x, -y)
            const Fq29 xPmQ = fq29_mul(fq29_add(fq29_sqr(lam), xPQ), one29);
            const Fq29 yPmQ = fq29_mul(fq29_sub(fq29_mul(lam, fq29_sub(xD, xPmQ)), yD), one29);
            // D stays in registers; the other three abscissae and the second ordinate wait in LDS (word-interleaved over the
            // lanes) and negations are formed when a point is taken: the walk then fits 256 registers without spilling.
#pragma unroll
            for (int l = 0; l < 14; ++l) {
                tab[0][l][threadIdx.x] = xQ.l[l];
                tab[1][l][threadIdx.x] = xPQ.l[l];
                tab[2][l][threadIdx.x] = xPmQ.l[l];
                tab[3][l][threadIdx.x] = yPmQ.l[l];
            }
        }
        for (int i = (int)jsf.len - 1; i >= 0; --i) {
            w = j29_double(w);
            const uint32_t dg = (jsf.dig[i >> 3] >> ((i & 7) * 4)) & 0xFu;    // (d1 + 1) | (d2 + 1) << 2, the same for every lane
            const int d1 = (int)(dg & 3u) - 1, d2 = (int)(dg >> 2) - 1;
            if (d1 == 0 && d2 == 0) continue;
            A29 t;
            bool negate;
            if (d2 == 0) { t.x = xD; t.y = yD; negate = d1 < 0; }
            else {
                const int xi = d1 == 0 ? 0 : (d1 == d2 ? 1 : 2);
#pragma unroll
                for (int l = 0; l < 14; ++l) t.x.l[l] = tab[xi][l][threadIdx.x];
                if (xi == 2) {
#pragma unroll
                    for (int l = 0; l < 14; ++l) t.y.l[l] = tab[3][l][threadIdx.x];
                    negate = d1 < 0;
                } else {
                    t.y = yD;
                    negate = xi == 0 ? d2 < 0 : d1 > 0;                          // D + phi(D) = (beta^2 x, -y)
                }
            }
            if (negate) t.y = fq29_neg(t.y);
            w = j29_add_mixed(w, t);
        }
        if (!inf1) w = j29_add_mixed(w, a1);
    }
    // back to affine: 1 / z batched over the lanes (the table in LDS is no longer needed)
    const bool has_z = fast && !w.inf;
    const Fq29 zi = block_inv64_29(has_z ? w.z : one29, inv_lds);
    if (fast) {
        A29 o;
        o.x = o.y = fq29_zero();
        if (has_z) {
            const Fq29 zi2 = fq29_sqr(zi);
            o.x = fq29_canon(fq29_mul(w.x, zi2));
            o.y = fq29_canon(fq29_mul(fq29_mul(w.y, zi2), zi));
        }
        new_gens[g] = o;
    } else if (general) {
        const uint32_t slot = atomicAdd(&special[0], 1u);
        special[1 + slot] = (uint32_t)g;
    }
}
// ---- the first round over prepared generators: a fixed-base comb per pair ----------------------------------------------------------
// The generators of an opening are public and fixed, so D_i = g_2i - g_2i+1 is known before any challenge is.  For each
// pair the prepared form holds the COMB_N = 2^COMB_A - 1 sums  E[m] = sum_{j : bit j of m} 2^(j COMB_W) D_i  as affine
// points.  With u = k1 + k2 lambda (k1, k2 < 2^128 <= 2^(COMB_A COMB_W)), position b of the comb takes bit j COMB_W + b
// of k1 for every tooth j as the index m1(b), likewise m2(b) from k2, and
//     [u] D = sum_b 2^b ( E[m1(b)] + phi(E[m2(b)]) ),   phi(x, y) = (beta x, y):
// COMB_W doublings and at most 2 COMB_W mixed additions instead of 129 doublings and ~65 additions, and no inversion for a
// table.  Every lane of the launch uses the same indices, so the table is laid out entry-major ([m][pair]): the lanes of a
// wave read consecutive points.
static constexpr int COMB_A = 8, COMB_W = 16, COMB_N = (1 << COMB_A) - 1;
static_assert(COMB_A * COMB_W >= 128, "the comb must cover 128-bit half scalars");
struct CombK { uint8_t m1[COMB_W + 2], m2[COMB_W + 2]; };
// No pair is special here: the table holds multiples of D whatever D is (infinity when the two generators are equal, a
// doubling when they are opposite), an entry at infinity is skipped, and the mixed addition itself handles a sum that
// meets its own operand.
// NT = 2 (the second round): the pair difference of that round is itself a fixed combination of prepared points,
//     g'_2j - g'_2j+1 = F_j + [u1] H_j,   F_j = g_4j+1 - g_4j+3,  H_j = (g_4j - g_4j+1) - (g_4j+2 - g_4j+3)
// (g'_i = g_2i+1 + [u1](g_2i - g_2i+1) are the first round's results, a missing generator is the point at infinity), so
//     g''_j = g'_2j+1 + [u2] F_j + [u1 u2] H_j:
// two combs that share their doublings, COMB_W doublings and at most 4 COMB_W additions instead of the 129-step walk.
struct CombItem { Fr* ns; A29* ng; const Fr* s; const A29* g; const A29* tab; const A29* tab2; Fr u_mont; CombK ck, ck2; };
struct CombBatch { CombItem it[OB_MAX]; };
template <int NT>
__global__ void __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_open_fold_comb(const CombBatch cb, size_t old_size, size_t new_size) {
    __shared__ int32_t inv_lds[14][2 * GT];
    Fr* __restrict__ new_scalars = cb.it[blockIdx.y].ns;
    A29* __restrict__ new_gens = cb.it[blockIdx.y].ng;
    const Fr* __restrict__ scalars = cb.it[blockIdx.y].s;
    const A29* __restrict__ A = cb.it[blockIdx.y].g;
    const A29* __restrict__ tab = cb.it[blockIdx.y].tab;
    const A29* __restrict__ tab2 = cb.it[blockIdx.y].tab2;
    const Fr u_mont = cb.it[blockIdx.y].u_mont;
    const CombK& ck = cb.it[blockIdx.y].ck;
    const CombK& ck2 = cb.it[blockIdx.y].ck2;
    const size_t g = (size_t)blockIdx.x * GT + threadIdx.x;
    const bool live = g < new_size;
    const size_t g0 = 2 * g, g1 = 2 * g + 1;
    const bool has1 = live && g1 < old_size;
    A29 a1;
    a1.x = a1.y = fq29_zero();
    if (has1) a1 = A[g1];
    if (live) {
        if (has1) new_scalars[g] = add(scalars[g0], mont_mul(u_mont, sub(scalars[g1], scalars[g0])));
        else new_scalars[g] = sub(scalars[g0], mont_mul(u_mont, scalars[g0]));
    }
    const bool inf1 = !has1 || a29_is_inf(a1);
    const bool fast = live;
    J29 w = j29_infinity();
    if (fast) {
        const Fq29 beta = fq29_from_fp(glv_beta());
        for (int b = COMB_W - 1; b >= 0; --b) {
            w = j29_double(w);
#pragma unroll
            for (int ti = 0; ti < NT; ++ti) {
                const A29* __restrict__ tb = ti ? tab2 : tab;
                const uint32_t m1 = ti ? ck2.m1[b] : ck.m1[b], m2 = ti ? ck2.m2[b] : ck.m2[b];          // the same for every lane
                if (m1) {
                    const A29 t = tb[(size_t)(m1 - 1) * new_size + g];
                    if (!a29_is_inf(t)) w = j29_add_mixed(w, t);
                }
                if (m2) {
                    A29 t = tb[(size_t)(m2 - 1) * new_size + g];
                    if (!a29_is_inf(t)) {
                        t.x = fq29_mul(t.x, beta);
                        w = j29_add_mixed(w, t);
                    }
                }
            }
        }
        if (!inf1) w = j29_add_mixed(w, a1);
    }
    const bool has_z = fast && !w.inf;
    const Fq29 zi = block_inv64_29(has_z ? w.z : fq29_one(), inv_lds);
    if (fast) {
        A29 o;
        o.x = o.y = fq29_zero();
        if (has_z) {
            const Fq29 zi2 = fq29_sqr(zi);
            o.x = fq29_canon(fq29_mul(w.x, zi2));
            o.y = fq29_canon(fq29_mul(fq29_mul(w.y, zi2), zi));
        }
        new_gens[g] = o;
    }
}
// ---- three rounds in one: the generators after the third fold straight from the prepared ones -------------------------------------
// When T0 and T1 of the first three rounds come from cross commitments of the opened tensor, nothing reads the generators of
// the second and third round but the next fold.  With c_b = prod_{k<3} (bit_k(b) ? 1 - u_k : u_k) (u_0 .. u_2 the three
// challenges; the c_b sum to one) the generators after three folds are
//     g^(3)_m = sum_{b<8} c_b g_(8m+b) = g_(8m+7) + sum_{b<7} [c_b] P_b,m,     P_b,m = g_(8m+b) - g_(8m+7),
// seven fixed-base combs that share their COMB_W doublings: at most 14 COMB_W additions per eight generators, where the
// three rounds one after the other take a comb per pair, a double comb per four and a 129-step walk per eight.
// Tables: [b][entry][m], built like the first round's.  The scalars are folded three times on the way.
static constexpr int JUMP_ROUNDS = 3, JUMP_SPAN = 1 << JUMP_ROUNDS, JUMP_TABS = JUMP_SPAN - 1;
struct JumpItem { Fr* ns; A29* ng; const Fr* s; const A29* g; const A29* tab; Fr u_mont[JUMP_ROUNDS]; CombK ck[JUMP_TABS]; };
struct JumpBatch { JumpItem it[OB_MAX]; };
__global__ void __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_open_fold_jump(const JumpBatch jb, size_t new_size) {
    __shared__ int32_t inv_lds[14][2 * GT];
    const JumpItem& it = jb.it[blockIdx.y];
    const size_t g = (size_t)blockIdx.x * GT + threadIdx.x;
    const bool live = g < new_size;
    A29 a1;
    a1.x = a1.y = fq29_zero();
    if (live) {
        a1 = it.g[JUMP_SPAN * g + JUMP_SPAN - 1];
        // the scalars, level by level as the rounds would fold them
        Fr v[JUMP_SPAN];
#pragma unroll
        for (int i = 0; i < JUMP_SPAN; ++i) v[i] = it.s[JUMP_SPAN * g + i];
#pragma unroll
        for (int k = 0; k < JUMP_ROUNDS; ++k)
#pragma unroll
            for (int i = 0; i < (JUMP_SPAN >> (k + 1)); ++i) v[i] = add(v[2 * i], mont_mul(it.u_mont[k], sub(v[2 * i + 1], v[2 * i])));
        it.ns[g] = v[0];
    }
    const bool inf1 = !live || a29_is_inf(a1);
    J29 w = j29_infinity();
    if (live) {
        const Fq29 beta = fq29_from_fp(glv_beta());
        for (int b = COMB_W - 1; b >= 0; --b) {
            w = j29_double(w);
            for (int ti = 0; ti < JUMP_TABS; ++ti) {
                const A29* __restrict__ tb = it.tab + (size_t)ti * COMB_N * new_size;
                const uint32_t m1 = it.ck[ti].m1[b], m2 = it.ck[ti].m2[b];          // the same for every lane
                if (m1) {
                    const A29 t = tb[(size_t)(m1 - 1) * new_size + g];
                    if (!a29_is_inf(t)) w = j29_add_mixed(w, t);
                }
                if (m2) {
                    A29 t = tb[(size_t)(m2 - 1) * new_size + g];
                    if (!a29_is_inf(t)) {
                        t.x = fq29_mul(t.x, beta);
                        w = j29_add_mixed(w, t);
                    }
                }
            }
        }
        if (!inf1) w = j29_add_mixed(w, a1);
    }
    const bool has_z = live && !w.inf;
    const Fq29 zi = block_inv64_29(has_z ? w.z : fq29_one(), inv_lds);
    if (live) {
        A29 o;
        o.x = o.y = fq29_zero();
        if (has_z) {
            const Fq29 zi2 = fq29_sqr(zi);
            o.x = fq29_canon(fq29_mul(w.x, zi2));
            o.y = fq29_canon(fq29_mul(fq29_mul(w.y, zi2), zi));
        }
        it.ng[g] = o;
    }
}
// the pairs k_open_fold29 left out, by the general Jacobian route in 32-bit limbs (one lane per pair, an inversion each)
__device__ __forceinline__ G1Affine a29_to_affine(const A29& p) {
    G1Affine r;
    r.x = fq29_to_fp(p.x); r.y = fq29_to_fp(p.y);
    return r;
}
struct SpecialBatch { A29* ng[OB_MAX]; const A29* g[OB_MAX]; const uint32_t* special[OB_MAX]; GlvK ku[OB_MAX]; };
__global__ void __launch_bounds__(GT) k_open_fold_special(const SpecialBatch sb, size_t old_size) {
    A29* __restrict__ new_gens = sb.ng[blockIdx.y];
    const A29* __restrict__ A = sb.g[blockIdx.y];
    const uint32_t* __restrict__ special = sb.special[blockIdx.y];
    const GlvK ku = sb.ku[blockIdx.y];
    const uint32_t count = special[0];
    for (uint32_t i = blockIdx.x * GT + threadIdx.x; i < count; i += gridDim.x * GT) {
        const size_t g = special[1 + i];
        const G1Affine a0 = a29_to_affine(A[2 * g]);
        const bool has1 = 2 * g + 1 < old_size;
        G1Affine a1;
        a1.x = a1.y = big_zero<12>();
        if (has1) a1 = a29_to_affine(A[2 * g + 1]);
        const bool inf1 = !has1 || aff_is_inf(a1);
        G1Jac diff = aff_to_jac(a0);
        if (!inf1) diff = g1_add_mixed(diff, g1_neg(a1));
        G1Jac r = g1_mul_glv(diff, ku);
        if (!inf1) r = g1_add_mixed(r, a1);
        A29 o;
        o.x = o.y = fq29_zero();
        if (!is_zero(r.z)) {
            const Fp zi = mont_inverse(r.z), zi2 = fp_sqr(zi);
            G1Affine af;
            af.x = fp_mul(r.x, zi2);
            af.y = fp_mul(fp_mul(r.y, zi2), zi);
            o = a29_from_affine(af);
            o.x = fq29_canon(o.x); o.y = fq29_canon(o.y);
        }
        new_gens[g] = o;
    }
}
// generator pairs' sums g_2i + g_2i+1 (an odd last element alone) for T of the first round; and the pairs' scalar sums
// negate: the differences g_2i - g_2i+1 instead (what the first round's comb is built on)
__global__ void __launch_bounds__(GT) k_open_pair_points(G1Jac* __restrict__ pj, const G1Affine* __restrict__ A, size_t old_size, size_t half_up, int negate) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= half_up) return;
    G1Jac p = aff_to_jac(A[2 * i]);
    if (2 * i + 1 < old_size) {
        G1Affine b = A[2 * i + 1];
        if (negate) b = g1_neg(b);
        if (!aff_is_inf(b)) p = g1_add_mixed(p, b);
    }
    pj[i] = p;
}
// out[j] = V[2j] - V[2j+1] over the points V[i] = A[off + i * stride], i < cnt (a missing one is the point at infinity)
__global__ void __launch_bounds__(GT) k_open_pair_diff(G1Jac* __restrict__ out, const G1Affine* __restrict__ A, size_t off, size_t stride, size_t cnt, size_t n_out) {
    const size_t j = (size_t)blockIdx.x * GT + threadIdx.x;
    if (j >= n_out) return;
    G1Jac p = g1_infinity();
    if (2 * j < cnt) p = aff_to_jac(A[off + 2 * j * stride]);
    if (2 * j + 1 < cnt) {
        const G1Affine b = g1_neg(A[off + (2 * j + 1) * stride]);
        if (!aff_is_inf(b)) p = g1_add_mixed(p, b);
    }
    out[j] = p;
}
// out[m] = A[m * span + b] - A[m * span + span - 1], m < n_out (the points of k_open_fold_jump's tables)
__global__ void __launch_bounds__(GT) k_open_span_diff(G1Jac* __restrict__ out, const G1Affine* __restrict__ A, uint32_t span, uint32_t b, size_t n_out) {
    const size_t m = (size_t)blockIdx.x * GT + threadIdx.x;
    if (m >= n_out) return;
    G1Jac p = aff_to_jac(A[m * span + b]);
    const G1Affine last = g1_neg(A[m * span + span - 1]);
    if (!aff_is_inf(last)) p = g1_add_mixed(p, last);
    out[m] = p;
}
struct PairBatch { Fr* ps[OB_MAX]; const Fr* s[OB_MAX]; };
__global__ void __launch_bounds__(256) k_open_pair_scalars(const PairBatch pb, size_t old_size, size_t half_up) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= half_up) return;
    Fr* __restrict__ ps = pb.ps[blockIdx.y];
    const Fr* __restrict__ scalars = pb.s[blockIdx.y];
    ps[i] = (2 * i + 1 < old_size) ? add(scalars[2 * i], scalars[2 * i + 1]) : scalars[2 * i];
}
__global__ void __launch_bounds__(GT) k_a29_to_jac(G1Jac* __restrict__ out, const A29* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * GT + threadIdx.x;
    if (i >= n) return;
    out[i] = a29_is_inf(in[i]) ? g1_infinity() : aff_to_jac(a29_to_affine(in[i]));
}
__global__ void __launch_bounds__(256) k_a29_canon(A29* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    A29 v = a[i];
    v.x = fq29_canon(v.x); v.y = fq29_canon(v.y);
    a[i] = v;
}
// ---- the last rounds in one batch ---------------------------------------------------------------------------------------
// Once n0 <= TAIL_N generators are left, every later round's generators are fixed linear combinations of these n0
// points: g at level j, block i, is sum over k in block i of W_j(k) g_k with W_j(k) = prod_{b<j} (bit_b(k) ? 1-u_b : u_b).
// So T, T0, T1 of all remaining rounds and the final generator are multi-scalar multiplications over the same n0
// affine points with coefficients that are plain field arithmetic; they run as one launch instead of a chain of
// rounds that each wait for a scalar multiplication.
// Folded scalars of all levels: level 0 is S itself, level j >= 1 sits at SL + sum_{1<=i<j} n_i, n_i = ceil(n0 / 2^i).
struct TailPtrs { Fr* SL[OB_MAX]; const Fr* S[OB_MAX]; };      // per opening of a batch (blockIdx.x of k_tail_scalars, blockIdx.y of k_tail_coeffs)
// U: the tail's challenges (Montgomery form), opening y's at U + y * ustride
// One workgroup per opening (the levels follow each other behind a barrier) of TAIL_SCALAR_T lanes: four waves find room on
// a compute unit whose SIMDs each hold a point kernel's waves; the sixteen of a 1024-lane workgroup waited milliseconds for it.
static constexpr int TAIL_SCALAR_T = 256;
__global__ void __launch_bounds__(TAIL_SCALAR_T) k_tail_scalars(const TailPtrs tp, const Fr* __restrict__ U, uint32_t ustride, uint32_t n0, uint32_t levels) {
    const Fr* __restrict__ usu = U + (size_t)blockIdx.x * ustride;
    const Fr* cur = tp.S[blockIdx.x];
    Fr* nxt = tp.SL[blockIdx.x];
    uint32_t n = n0;
    for (uint32_t j = 0; j < levels; ++j) {
        const uint32_t ns = (n + 1) / 2;
        for (uint32_t g = threadIdx.x; g < ns; g += TAIL_SCALAR_T) {
            const Fr s0 = cur[2 * g];
            nxt[g] = (2 * g + 1 < n) ? add(s0, mont_mul(usu[j], sub(cur[2 * g + 1], s0))) : sub(s0, mont_mul(usu[j], s0));
        }
        __syncthreads();
        cur = nxt;
        nxt += ns;
        n = ns;
    }
}
// C[(3j+0)*n0 + k] = s_j[k>>j] W_j(k); C[(3j+1)*n0 + k] = s_j[(k>>j)-1] W_j(k) for odd k>>j; C[(3j+2)*n0 + k] = s_j[(k>>j)+1] W_j(k)
// for even k>>j with a partner; zero elsewhere.  C[3*levels*n0 + k] = W_levels(k).
__global__ void __launch_bounds__(256) k_tail_coeffs(Fr* __restrict__ C0, const TailPtrs tp, const Fr* __restrict__ U, uint32_t ustride, uint32_t n0, uint32_t levels) {
    const uint32_t k = blockIdx.x * 256 + threadIdx.x;
    if (k >= n0) return;
    const Fr* __restrict__ usu = U + (size_t)blockIdx.y * ustride;
    Fr* __restrict__ C = C0 + (size_t)blockIdx.y * (3 * levels + 1) * n0;
    const Fr* __restrict__ SL = tp.SL[blockIdx.y];
    const Fr* __restrict__ S = tp.S[blockIdx.y];
    const Fr one_m = big_one_mont<8>();
    Fr W = one_m;                 // Montgomery form
    const Fr* sj = S;
    const Fr* nxt = SL;
    uint32_t n = n0;
    const Fr zero = big_zero<8>();
    for (uint32_t j = 0; j < levels; ++j) {
        const uint32_t i = k >> j;
        // mont_mul(Montgomery W, standard s) is the standard-form product
        C[(size_t)(3 * j) * n0 + k] = mont_mul(W, sj[i]);
        C[(size_t)(3 * j + 1) * n0 + k] = (i & 1u) ? mont_mul(W, sj[i - 1]) : zero;
        C[(size_t)(3 * j + 2) * n0 + k] = (!(i & 1u) && i + 1 < n) ? mont_mul(W, sj[i + 1]) : zero;
        W = mont_mul(W, (i & 1u) ? sub(one_m, usu[j]) : usu[j]);
        const uint32_t ns = (n + 1) / 2;
        sj = nxt;
        nxt += ns;
        n = ns;
    }
    C[(size_t)(3 * levels) * n0 + k] = from_mont(W);
}
__global__ void __launch_bounds__(64) k_u32_zero(uint32_t* __restrict__ p, uint32_t n, size_t stride) {      // p[i * stride] = 0, i < n
    for (uint32_t i = threadIdx.x; i < n; i += 64) p[(size_t)i * stride] = 0u;
}
// after the last round of an opening without a batched tail: the folded generator is the last proof point
__global__ void __launch_bounds__(GT) k_open_finish(G1Jac* __restrict__ pts, const A29* __restrict__ last_gen, uint32_t rounds) {
    if (blockIdx.x == 0 && threadIdx.x == 0) pts[3 * rounds] = a29_is_inf(last_gen[0]) ? g1_infinity() : aff_to_jac(a29_to_affine(last_gen[0]));
}

// ---- host side ----------------------------------------------------------------------------------------------------------
static inline Fr load_fr(const uint32_t* p) { Fr r; memcpy(&r, p, 32); return r; }
static inline G1Jac load_g1(const uint32_t* p) { G1Jac r; memcpy(&r, p, 144); return r; }

#define GLAUNCH(kernel, n, st, ...)                                                                          \
    do {                                                                                                     \
        if ((n) > 0) {                                                                                       \
            hipLaunchKernelGGL(kernel, dim3(cdiv((n), GT)), dim3(GT), 0, (hipStream_t)(st), __VA_ARGS__);     \
            ZK_LAUNCH_CHECK();                                                                               \
        }                                                                                                    \
    } while (0)

// sum of n points at `in` into one point at `out` (device); `in` is not modified
static int g1_sum_device(G1Jac* out, const G1Jac* in, size_t n, hipStream_t st) {
    if (n == 0) {
        G1Jac inf = g1_infinity();
        hipLaunchKernelGGL(k_g1_fill, dim3(1), dim3(GT), 0, st, out, inf, (size_t)1);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    uint32_t nseg = (uint32_t)((n + 4 * GT - 1) / (4 * GT));
    if (nseg > 1024) nseg = 1024;
    if (nseg <= 1) {
        hipLaunchKernelGGL(k_g1_rowsum, dim3(1, 1), dim3(GT), 0, st, out, in, n, 1u);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    Scratch part(sizeof(G1Jac) * nseg, st);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_g1_rowsum, dim3(1, nseg), dim3(GT), 0, st, part.as<G1Jac>(), in, n, nseg);
    hipLaunchKernelGGL(k_g1_rowsum, dim3(1, 1), dim3(GT), 0, st, out, part.as<G1Jac>(), (size_t)nseg, 1u);
    ZK_LAUNCH_CHECK();
    return 0;
}

// Optional timing of the fold kernel's launches with events on its own stream (measurement only).
struct FoldTimer {
    std::mutex mu;
    bool on = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> ev;
    double fp_mults = 0;      // Fp multiplications the timed launches perform by the formulas' count
    unsigned long long pairs = 0;
    // the same per method: 0 the walk (k_open_fold29), 1 the one- and two-table combs (k_open_fold_comb), 2 the three-round fold (k_open_fold_jump)
    std::vector<int> method;
    double m_mults[3] = {0, 0, 0};
    unsigned long long m_pairs[3] = {0, 0, 0};
};
static FoldTimer g_fold_timer;
static const int g_fold_timer_hook = (at_shutdown([] {
    std::lock_guard<std::mutex> lk(g_fold_timer.mu);
    for (auto& e : g_fold_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    g_fold_timer.ev.clear();
    g_fold_timer.on = false;
}), 0);
// Fp multiplications of one pair of the fold by the formulas' count (two 8-limb products aside)
static double fold_fp_mults_per_pair(const JsfK& j) {
    int adds = 0;
    for (uint32_t i = 0; i < j.len; ++i) adds += (((j.dig[i >> 3] >> ((i & 7) * 4)) & 0xFu) != 5u) ? 1 : 0;    // 5 = both digits zero
    // difference (4), its share of two batched inversions (6), table (7), doublings (7 each), mixed additions (11 each), final addition (11)
    return 4.0 + 6.0 + 7.0 + 7.0 * j.len + 11.0 * adds + 11.0;
}

// u = k1 + k2 * lambda with 0 <= k1 < lambda and k2 <= lambda + 1 (r = lambda^2 + lambda + 1): one long division
static GlvK glv_split(const Fr& u) {
    const unsigned __int128 lam = ((unsigned __int128)0xac45a4010001a402ull << 64) | 0x00000000ffffffffull;
    unsigned __int128 rem = 0, q = 0;
    for (int i = 255; i >= 0; --i) {
        const bool top = (rem >> 127) != 0;
        rem = (rem << 1) | ((u.v[i >> 5] >> (i & 31)) & 1u);
        q <<= 1;
        if (top || rem >= lam) { rem -= lam; q |= 1; }
    }
    GlvK k;
    for (int i = 0; i < 4; ++i) { k.k1[i] = (uint32_t)(rem >> (32 * i)); k.k2[i] = (uint32_t)(q >> (32 * i)); }
    return k;
}
// joint sparse form of the two halves of a split scalar (Solinas): the fewest non-zero digit pairs among signed binary forms
static JsfK jsf_of(const GlvK& k) {
    unsigned __int128 a = 0, b = 0;
    for (int i = 3; i >= 0; --i) { a = (a << 32) | k.k1[i]; b = (b << 32) | k.k2[i]; }
    JsfK out;
    memset(&out, 0, sizeof(out));
    unsigned d1 = 0, d2 = 0, len = 0;
    while (a + d1 > 0 || b + d2 > 0) {
        const unsigned l1 = (unsigned)((a & 7) + d1) & 7u, l2 = (unsigned)((b & 7) + d2) & 7u;
        int u1 = 0, u2 = 0;
        if (l1 & 1u) { u1 = 2 - (int)(l1 & 3u); if ((l1 == 3 || l1 == 5) && (l2 & 3u) == 2) u1 = -u1; }
        if (l2 & 1u) { u2 = 2 - (int)(l2 & 3u); if ((l2 == 3 || l2 == 5) && (l1 & 3u) == 2) u2 = -u2; }
        if (2 * (int)d1 == 1 + u1) d1 = 1 - d1;
        if (2 * (int)d2 == 1 + u2) d2 = 1 - d2;
        a >>= 1;
        b >>= 1;
        out.dig[len >> 3] |= (uint32_t)((u1 + 1) | ((u2 + 1) << 2)) << ((len & 7) * 4);
        ++len;
    }
    out.len = len;
    return out;
}

// The generators of an opening in the form its rounds work on: A29 points, and behind them the pair sums
// g_2i + g_2i+1 that T of the first round is summed over (n + ceil(n/2) points in one array).  Nothing in it depends on
// what is opened, so a caller that opens against the same generators again keeps it (zk_g1_open_prepare).
static int open_prep_build(A29* out, const G1Jac* gens, size_t n, Arena& arena, hipStream_t st) {
    const size_t half_up = (n + 1) / 2;
    Scratch& aff = arena.add(sizeof(G1Affine) * n);
    Scratch& pj = arena.add(sizeof(G1Jac) * half_up);
    Scratch& paff = arena.add(sizeof(G1Affine) * half_up);
    if (aff.rc || pj.rc || paff.rc) return aff.rc ? aff.rc : (pj.rc ? pj.rc : paff.rc);
    hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(n, CH), GT)), dim3(GT), 0, st, aff.p, gens, n);
    hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(n, 256)), dim3(256), 0, st, out, aff.as<G1Affine>(), n);
    hipLaunchKernelGGL(k_open_pair_points, dim3(cdiv(half_up, GT)), dim3(GT), 0, st, pj.as<G1Jac>(), aff.as<G1Affine>(), n, half_up, 0);
    hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(half_up, CH), GT)), dim3(GT), 0, st, paff.p, pj.as<G1Jac>(), half_up);
    hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(half_up, 256)), dim3(256), 0, st, out + n, paff.as<G1Affine>(), half_up);
    ZK_LAUNCH_CHECK();
    return 0;
}

// Queues one round: the scalars' digits and the fold on st, the bucket sums on aux.  gens: the round's generators (A29);
// with_T (the first round): the pair sums follow them at gens + old_size.  wsum_round: the round's 3 x MW window sums
// (T, T0, T1); without with_T the first MW are left alone (T of that round then comes from k_open_chain).
// Round 0 needs T = sum_j s_j g_j over all generators besides T0 and T1.  With the pairs' sums,
//   sum_i (s_2i + s_2i+1)(g_2i + g_2i+1) = T + T0 + T1,
// so T costs a bucket sum over half as many points: pair i gets the scalar s_2i + s_2i+1 (mod r: the generators have
// order r) and the point g_2i + g_2i+1; an odd last element stands alone.  k_open_t_fix takes T0 and T1 off again,
// window by window.
__global__ void __launch_bounds__(64) k_open_t_fix(G1Jac* __restrict__ wsum0, uint32_t item_stride) {
    const uint32_t w = threadIdx.x;
    if (w >= (uint32_t)MW) return;
    G1Jac* __restrict__ wsum = wsum0 + (size_t)blockIdx.x * item_stride;
    wsum[w] = g1_add(g1_add(wsum[w], g1_neg(wsum[MW + w])), g1_neg(wsum[2 * MW + w]));
}
// One round of `count` openings of equal size (count <= OB_MAX): one launch of each kernel covers all of them.
// comb: the first round's table; comb2 (second round): the tables of F and H one after the other, u_prev the first round's challenge
struct RoundItem { Fr* new_scalars; A29* new_gens; const Fr* scalars; const A29* gens; Fr u; const A29* comb = nullptr; const A29* comb2 = nullptr; Fr u_prev = Fr(); };
// Fp multiplications of one pair of the comb fold by the formulas' count
static double comb_fp_mults_per_pair(const CombK& ck, const CombK* ck2 = nullptr) {
    int adds = 0, phis = 0;
    for (int b = 0; b < COMB_W; ++b) { adds += (ck.m1[b] ? 1 : 0) + (ck.m2[b] ? 1 : 0); phis += ck.m2[b] ? 1 : 0; }
    if (ck2) for (int b = 0; b < COMB_W; ++b) { adds += (ck2->m1[b] ? 1 : 0) + (ck2->m2[b] ? 1 : 0); phis += ck2->m2[b] ? 1 : 0; }
    // doublings (7 each), mixed additions (11 each), the endomorphism's product, final addition (11), its share of one batched inversion (3) and the way back to affine (5)
    return 7.0 * COMB_W + 11.0 * adds + phis + 11.0 + 3.0 + 5.0;
}
static CombK comb_of(const GlvK& k) {
    CombK ck;
    memset(&ck, 0, sizeof(ck));
    for (int b = 0; b < COMB_W; ++b)
        for (int j = 0; j < COMB_A; ++j) {
            const int bit = j * COMB_W + b;
            if (bit >= 128) continue;
            ck.m1[b] |= (uint8_t)(((k.k1[bit >> 5] >> (bit & 31)) & 1u) << j);
            ck.m2[b] |= (uint8_t)(((k.k2[bit >> 5] >> (bit & 31)) & 1u) << j);
        }
    return ck;
}
// given: what of this round's sums comes from commitments of the tensor's rows (open_cross_sums_queue) and is not summed here:
// 0 nothing, 1 T of the first round (no pair sums), 2 T0 and T1 as well (no bucket sums at all: the round is its fold)
// later (optional): the reductions of this round's raw buckets are appended to it instead of launched (the caller runs them
// all at once behind its last round); a round whose T comes from the pair sums (k_open_t_fix) reduces at once
static int open_round_launch(const RoundItem* items, int count, size_t old_size, bool with_T, int given, G1Jac* wsum_round, uint32_t wsum_item_stride, Arena& arena,
                             hipStream_t st, hipStream_t aux, std::vector<hipEvent_t>& events, std::vector<PointDesc>* later = nullptr) {
    ZK_ARG(old_size < (1ull << 31), "opening: more than 2^31 generators");
    ZK_ARG(count >= 1 && count <= OB_MAX, "opening: bad batch size");
    const size_t new_size = (old_size + 1) / 2;
    const bool chained = !with_T || given >= 1;
    if (given < 2) {
    const size_t dig_bytes = (size_t)(MW + 1) * old_size;
    Scratch& dig = arena.add(dig_bytes * count);
    if (dig.rc) return dig.rc;
    {
        RecodeBatch rb;
        for (int i = 0; i < OB_MAX; ++i) { rb.D[i] = dig.as<int8_t>() + dig_bytes * (i < count ? i : 0); rb.S[i] = items[i < count ? i : 0].scalars; }
        hipLaunchKernelGGL(k_msm_recode, dim3(cdiv(old_size, 256), count), dim3(256), 0, st, rb, old_size);
        ZK_LAUNCH_CHECK();
    }
    if (aux != st) {
        hipEvent_t ready;
        ZK_HIP(hipEventCreateWithFlags(&ready, hipEventDisableTiming));
        events.push_back(ready);
        ZK_HIP(hipEventRecord(ready, st));
        ZK_HIP(hipStreamWaitEvent(aux, ready, 0));
    }
    // ---- side chain (aux): bucket sums, window sums; nothing here feeds the next fold ----
    MsmDescs<OB_SUMS> descs;
    const uint32_t half = (uint32_t)(old_size / 2);
    const uint32_t half_up = (uint32_t)new_size;
    const uint32_t n_per = chained ? 2u : 3u, n_msm = n_per * (uint32_t)count;
    const uint32_t ds = (uint32_t)old_size;
    const int8_t* dig2p = nullptr;
    const size_t dig2_bytes = (size_t)(MW + 1) * half_up;
    if (!chained) {
        Scratch& ps = arena.add(sizeof(Fr) * half_up * count);
        Scratch& dig2 = arena.add(dig2_bytes * count);
        if (ps.rc || dig2.rc) return ps.rc ? ps.rc : dig2.rc;
        PairBatch pb;
        RecodeBatch rb;
        for (int i = 0; i < OB_MAX; ++i) {
            const int k = i < count ? i : 0;
            pb.ps[i] = ps.as<Fr>() + (size_t)half_up * k; pb.s[i] = items[k].scalars;
            rb.D[i] = dig2.as<int8_t>() + dig2_bytes * k; rb.S[i] = pb.ps[i];
        }
        hipLaunchKernelGGL(k_open_pair_scalars, dim3(cdiv(half_up, 256), count), dim3(256), 0, aux, pb, old_size, (size_t)half_up);
        hipLaunchKernelGGL(k_msm_recode, dim3(cdiv(half_up, 256), count), dim3(256), 0, aux, rb, (size_t)half_up);
        dig2p = dig2.as<int8_t>();
    }
    uint32_t q = 0;
    for (int i = 0; i < count; ++i) {
        const int8_t* dg = dig.as<int8_t>() + dig_bytes * i;
        if (!chained) descs.d[q++] = MsmDesc{dig2p + dig2_bytes * i, items[i].gens, half_up, half_up, 1u, 0u, 1u, (uint32_t)old_size, 0u};
        descs.d[q++] = MsmDesc{dg, items[i].gens, ds, half, 2u, 0u, 2u, 1u, 1u};
        descs.d[q++] = MsmDesc{dg, items[i].gens, ds, half, 2u, 1u, 2u, 0u, 2u};
    }
    for (; q < (uint32_t)OB_SUMS; ++q) descs.d[q] = MsmDesc{dig.as<int8_t>(), items[0].gens, ds, 0u, 1u, 0u, 1u, 0u, 0u};
    // One chunk per workgroup: many short workgroups keep every compute unit busy to the end of the launch (with few
    // long ones, all equally long, whatever does not fit the first turn waits a whole turn); the raw buckets of the
    // segments are summed afterwards.  Very large inputs take more chunks per workgroup to bound the bucket storage.
    const size_t count_max = chained ? half : half_up;
    const uint32_t chunks = count_max ? cdiv(count_max, MSEG) : 1u;
    const uint32_t cps = (chunks + 255u) / 256u;
    const uint32_t nseg = (chunks + cps - 1) / cps;
    Scratch& partial = arena.add(sizeof(G1Jac) * n_msm * MW * (size_t)nseg * MT);
    if (partial.rc) return partial.rc;
    G1Jac* wsum = wsum_round + (size_t)(3 - n_per) * MW;
    hipLaunchKernelGGL(k_msm_seg<OB_SUMS>, dim3(nseg, MW, n_msm), dim3(MSL), 0, aux, partial.as<G1Jac>(), descs, (const MsmDesc*)nullptr, nseg, cps);
    {
        // sum the segments' raw buckets eight at a time (a lane per bucket and window: the reduction, one workgroup per sum,
        // then walks single buckets), then weight and total
        const G1Jac* cur = partial.as<G1Jac>();
        uint32_t ns = nseg;
        while (ns > 1) {
            const uint32_t ng = (ns + 7) / 8;
            Scratch& nxt = arena.add(sizeof(G1Jac) * n_msm * MW * (size_t)ng * MT);
            if (nxt.rc) return nxt.rc;
            hipLaunchKernelGGL(k_msm_bucket_fold, dim3(n_msm * MW, ng), dim3(MT), 0, aux, nxt.as<G1Jac>(), cur, ns);
            cur = nxt.as<G1Jac>();
            ns = ng;
        }
        if (later && chained) {
            for (uint32_t z = 0; z < n_msm; ++z)
                later->push_back(PointDesc{cur + (size_t)z * MW * ns * MT, wsum + (size_t)(z / n_per) * wsum_item_stride + (size_t)(z % n_per) * MW, ns, 0u});
        } else hipLaunchKernelGGL(k_msm_point, dim3(n_msm), dim3(MT), 0, aux, wsum, (G1Jac*)nullptr, (const MsmDesc*)nullptr, cur, ns, n_per, wsum_item_stride, (const PointDesc*)nullptr);
    }
    if (!chained) hipLaunchKernelGGL(k_open_t_fix, dim3(count), dim3(64), 0, aux, wsum, wsum_item_stride);
    ZK_LAUNCH_CHECK();
    }
    // ---- critical chain (st): the fold ----
    const size_t sp_stride = 1 + new_size;
    Scratch& special = arena.add(sizeof(uint32_t) * sp_stride * count);
    if (special.rc) return special.rc;
    bool use_comb = with_T, use_comb2 = !with_T;
    for (int i = 0; i < count; ++i) { use_comb = use_comb && items[i].comb != nullptr; use_comb2 = use_comb2 && items[i].comb2 != nullptr; }
    FoldBatch fb;
    CombBatch cbt;
    SpecialBatch sb;
    double fp_mults = 0;
    for (int i = 0; i < OB_MAX; ++i) {
        const int k = i < count ? i : 0;
        const GlvK ku = glv_split(items[k].u);
        uint32_t* sp = special.as<uint32_t>() + sp_stride * k;
        if (use_comb || use_comb2) {
            CombItem& f = cbt.it[i];
            f.ns = items[k].new_scalars; f.ng = items[k].new_gens; f.s = items[k].scalars; f.g = items[k].gens;
            f.u_mont = to_mont(items[k].u);
            f.ck = comb_of(ku);
            if (use_comb) {
                f.tab = items[k].comb; f.tab2 = items[k].comb;
                f.ck2 = f.ck;
                if (i < count) fp_mults += comb_fp_mults_per_pair(f.ck) * (double)new_size;
            } else {
                f.tab = items[k].comb2; f.tab2 = items[k].comb2 + (size_t)COMB_N * new_size;
                // [u2] of [u1] H is [u1 u2 mod r] H: the generators have order r
                f.ck2 = comb_of(glv_split(from_mont(mont_mul(to_mont(items[k].u_prev), to_mont(items[k].u)))));
                if (i < count) fp_mults += comb_fp_mults_per_pair(f.ck, &f.ck2) * (double)new_size;
            }
        } else {
            FoldItem& f = fb.it[i];
            f.ns = items[k].new_scalars; f.ng = items[k].new_gens; f.s = items[k].scalars; f.g = items[k].gens; f.special = sp;
            f.u_mont = to_mont(items[k].u);
            f.jsf = jsf_of(ku);
            if (i < count) fp_mults += fold_fp_mults_per_pair(f.jsf) * (double)new_size;
        }
        sb.ng[i] = items[k].new_gens; sb.g[i] = items[k].gens; sb.special[i] = sp; sb.ku[i] = ku;
    }
    hipLaunchKernelGGL(k_u32_zero, dim3(1), dim3(64), 0, st, special.as<uint32_t>(), (uint32_t)count, sp_stride);
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (g_fold_timer.on) {
        ZK_HIP(hipEventCreate(&t0));
        ZK_HIP(hipEventCreate(&t1));
        ZK_HIP(hipEventRecord(t0, st));
    }
    if (use_comb) hipLaunchKernelGGL(k_open_fold_comb<1>, dim3(cdiv(new_size, GT), count), dim3(GT), 0, st, cbt, old_size, new_size);
    else if (use_comb2) hipLaunchKernelGGL(k_open_fold_comb<2>, dim3(cdiv(new_size, GT), count), dim3(GT), 0, st, cbt, old_size, new_size);
    else hipLaunchKernelGGL(k_open_fold29, dim3(cdiv(new_size, GT), count), dim3(GT), 0, st, fb, old_size, new_size);
    if (g_fold_timer.on) {
        ZK_HIP(hipEventRecord(t1, st));
        std::lock_guard<std::mutex> lk(g_fold_timer.mu);
        g_fold_timer.ev.emplace_back(t0, t1);
        g_fold_timer.fp_mults += fp_mults;
        g_fold_timer.pairs += new_size * (size_t)count;
        const int mth = (use_comb || use_comb2) ? 1 : 0;
        g_fold_timer.method.push_back(mth);
        g_fold_timer.m_mults[mth] += fp_mults;
        g_fold_timer.m_pairs[mth] += new_size * (size_t)count;
    }
    hipLaunchKernelGGL(k_open_fold_special, dim3(16, count), dim3(GT), 0, st, sb, old_size);
    ZK_LAUNCH_CHECK();
    return 0;
}

// Queues the batch for the last `levels` rounds (rounds r0 .. r0+levels-1 of `rounds`) over n0 <= TAIL_N generators.
// Writes T, T0, T1 of those rounds and the final generator into pts; *final_scalar points at the folded scalar.
// Challenges and bucket-sum descriptors of a job travel through one pinned host buffer of 64 KiB (held until the job
// ends) into one device block: the challenges of all openings (Montgomery form, `rounds` per opening) in its first half, the
// descriptors of the batched last rounds in its second.
static constexpr size_t JOB_U_BYTES = 32768, JOB_DESC_BYTES = 32768;
static int open_tail_launch(const Fr** scalars, const A29* const* gens, int count, size_t n0, int levels, int r0, int rounds, G1Jac* pts, const Fr* U_dev, void* pin_host,
                            void* desc_dev, Arena& arena, hipStream_t st) {
    const int n_msm = 3 * levels + 1;
    const int total = n_msm * count;
    ZK_ARG(sizeof(MsmDesc) * (size_t)total <= JOB_DESC_BYTES, "opening: too many sums in the batched last rounds");
    const size_t npts = 3 * (size_t)rounds + 1;
    const size_t sl_n = n0 + (size_t)levels + 1;
    Scratch& sl = arena.add(sizeof(Fr) * sl_n * count);
    const uint32_t nseg = cdiv(n0, MSEG), cps = 1;       // one chunk per workgroup, as in the halving rounds
    const size_t ncoef = (size_t)n_msm * n0 * count;
    Scratch& coef = arena.add(sizeof(Fr) * ncoef);
    Scratch& partial = arena.add(sizeof(G1Jac) * total * MW * (size_t)nseg * MT);
    Scratch& dig = arena.add((size_t)(MW + 1) * ncoef);
    if (sl.rc) return sl.rc;
    if (coef.rc) return coef.rc;
    if (partial.rc) return partial.rc;
    if (dig.rc) return dig.rc;
    ZK_ARG(ncoef < (1ull << 32), "opening: batched last rounds too large");
    TailPtrs tp;
    for (int i = 0; i < OB_MAX; ++i) { const int k = i < count ? i : 0; tp.SL[i] = sl.as<Fr>() + sl_n * k; tp.S[i] = scalars[k]; }
    hipLaunchKernelGGL(k_tail_scalars, dim3(count), dim3(TAIL_SCALAR_T), 0, st, tp, U_dev + r0, (uint32_t)rounds, (uint32_t)n0, (uint32_t)levels);
    hipLaunchKernelGGL(k_tail_coeffs, dim3(cdiv(n0, 256), count), dim3(256), 0, st, coef.as<Fr>(), tp, U_dev + r0, (uint32_t)rounds, (uint32_t)n0, (uint32_t)levels);
    {
        RecodeBatch rb;
        for (int i = 0; i < OB_MAX; ++i) { rb.D[i] = dig.as<int8_t>(); rb.S[i] = coef.as<Fr>(); }
        hipLaunchKernelGGL(k_msm_recode, dim3(cdiv(ncoef, 256), 1), dim3(256), 0, st, rb, ncoef);
    }
    MsmDesc* hd = reinterpret_cast<MsmDesc*>((char*)pin_host + JOB_U_BYTES);
    for (int it = 0; it < count; ++it)
        for (int i = 0; i < n_msm; ++i) {
            const uint32_t slot = (uint32_t)(npts * it) + (i == 3 * levels ? 3u * (uint32_t)rounds : 3u * (uint32_t)r0 + (uint32_t)i);
            hd[it * n_msm + i] = MsmDesc{dig.as<int8_t>(), gens[it], (uint32_t)ncoef, (uint32_t)n0, 1u, (uint32_t)(((size_t)it * n_msm + i) * n0), 1u, 0u, slot};
        }
    ZK_HIP(hipMemcpyAsync(desc_dev, hd, sizeof(MsmDesc) * (size_t)total, hipMemcpyHostToDevice, st));
    const MsmDesc* dd = (const MsmDesc*)desc_dev;
    hipLaunchKernelGGL(k_msm_seg<1>, dim3(nseg, MW, total), dim3(MSL), 0, st, partial.as<G1Jac>(), MsmDescs<1>(), dd, nseg, cps);
    hipLaunchKernelGGL(k_msm_point, dim3(total), dim3(MT), 0, st, (G1Jac*)nullptr, pts, dd, partial.as<G1Jac>(), nseg, 1u, 0u, (const PointDesc*)nullptr);
    ZK_LAUNCH_CHECK();
    // the folded scalar is the single element of the last level
    size_t off = 0, nn = n0;
    for (int j = 1; j < levels; ++j) { nn = (nn + 1) / 2; off += nn; }
    for (int it = 0; it < count; ++it) scalars[it] = sl.as<Fr>() + sl_n * it + off;
    return 0;
}

extern "C" {

int zk_g1_fill(void* out, const uint32_t* point, size_t n, void* st) { GLAUNCH(k_g1_fill, n, st, (G1Jac*)out, load_g1(point), n); return 0; }
int zk_g1_neg(void* out, const void* a, size_t n, void* st) { GLAUNCH(k_g1_neg, n, st, (G1Jac*)out, (const G1Jac*)a, n); return 0; }
int zk_g1_affine_neg(void* out, const void* a, size_t n, void* st) { GLAUNCH(k_g1aff_neg, n, st, (G1Affine*)out, (const G1Affine*)a, n); return 0; }
int zk_g1_affine_to_jacobian(void* out, const void* a, size_t n, void* st) { GLAUNCH(k_g1aff_to_jac, n, st, (G1Jac*)out, (const G1Affine*)a, n); return 0; }
// out[i] = a[i] +/- b[i or 0]; b_count is n (elementwise) or 1 (broadcast, b on the device)
int zk_g1_add(void* out, const void* a, const void* b, size_t n, size_t b_count, int subtract, void* st) {
    ZK_ARG(b_count == n || b_count == 1, "zk_g1_add: b_count must be n or 1");
    GLAUNCH(k_g1_add, n, st, (G1Jac*)out, (const G1Jac*)a, (const G1Jac*)b, n, b_count, subtract);
    return 0;
}
int zk_g1_madd(void* out, const void* a, const void* b_affine, size_t n, size_t b_count, int subtract, void* st) {
    ZK_ARG(b_count == n || b_count == 1, "zk_g1_madd: b_count must be n or 1");
    GLAUNCH(k_g1_madd, n, st, (G1Jac*)out, (const G1Jac*)a, (const G1Affine*)b_affine, n, b_count, subtract);
    return 0;
}
int zk_g1_scalar_mul(void* out, const void* g, const void* s, size_t ng, size_t n, void* st) {
    ZK_ARG(ng >= 1 || n == 0, "zk_g1_scalar_mul: no generators");
    GLAUNCH(k_g1_scalar_mul, n, st, (G1Jac*)out, (const G1Jac*)g, (const Fr*)s, ng, n);
    return 0;
}
int zk_g1_sum(uint32_t* out_host, const void* a, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    Scratch res(sizeof(G1Jac), st);
    if (res.rc) return res.rc;
    int rc = g1_sum_device(res.as<G1Jac>(), (const G1Jac*)a, n, st);
    if (rc) return rc;
    void* stage = nullptr;
    rc = staging(&stage, sizeof(G1Jac));
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, res.p, sizeof(G1Jac), hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    memcpy(out_host, stage, sizeof(G1Jac));
    return 0;
}
int zk_g1_rowwise_sum(void* out, const void* in, size_t nrow, size_t ncol, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (nrow == 0) return 0;
    ZK_ARG(ncol >= 1, "zk_g1_rowwise_sum: ncol == 0");
    ZK_ARG(nrow <= 0x7fffffffu, "zk_g1_rowwise_sum: too many rows");
    uint32_t nseg = 1;
    if (nrow < 1024 && ncol > 8 * GT) { nseg = (uint32_t)(ncol / (4 * GT)); if (nseg > 64) nseg = 64; if (nseg < 1) nseg = 1; }
    if (nseg == 1) {
        hipLaunchKernelGGL(k_g1_rowsum, dim3((unsigned)nrow, 1), dim3(GT), 0, st, (G1Jac*)out, (const G1Jac*)in, ncol, 1u);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    Scratch part(sizeof(G1Jac) * nrow * nseg, st);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_g1_rowsum, dim3((unsigned)nrow, nseg), dim3(GT), 0, st, part.as<G1Jac>(), (const G1Jac*)in, ncol, nseg);
    hipLaunchKernelGGL(k_g1_rowsum, dim3((unsigned)nrow, 1), dim3(GT), 0, st, (G1Jac*)out, part.as<G1Jac>(), (size_t)nseg, 1u);
    ZK_LAUNCH_CHECK();
    return 0;
}
// G1TensorJacobian::operator()(u) (g1-tensor.cu:500-514); out_host receives one point
int zk_g1_me(uint32_t* out_host, const void* a, size_t n, const uint32_t* u, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(n >= 1, "zk_g1_me: empty tensor");
    const G1Jac* cur = (const G1Jac*)a;
    size_t cur_n = n;
    void* bufs[2] = {nullptr, nullptr};
    int which = 0, rc = 0;
    for (int lvl = 0; lvl < k && rc == 0; ++lvl) {
        const size_t out_n = (cur_n + 1) / 2;
        if (!bufs[which]) rc = pool_alloc(&bufs[which], sizeof(G1Jac) * out_n, st);
        if (rc) break;
        const Fr x = from_mont(load_fr(u + 8 * lvl));   // the reference passes unmont(u) to the scalar multiplication
        hipLaunchKernelGGL(k_g1_me_step, dim3(cdiv(out_n, GT)), dim3(GT), 0, st, (G1Jac*)bufs[which], cur, x, cur_n, out_n);
        if (hipGetLastError() != hipSuccess) { rc = hip_fail(hipErrorLaunchFailure, "k_g1_me_step", __FILE__, __LINE__); break; }
        cur = (const G1Jac*)bufs[which];
        cur_n = out_n;
        which ^= 1;
    }
    if (rc == 0) {
        void* stage = nullptr;
        rc = staging(&stage, sizeof(G1Jac));
        if (rc == 0) {
            hipError_t e = hipMemcpyAsync(stage, cur, sizeof(G1Jac), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess) e = hipStreamSynchronize(st);
            if (e != hipSuccess) rc = hip_fail(e, "zk_g1_me copy", __FILE__, __LINE__);
            else memcpy(out_host, stage, sizeof(G1Jac));
        }
    }
    for (int i = 0; i < 2; ++i) if (bufs[i]) pool_free(bufs[i], st);
    return rc;
}
// canonical form: z = ONE (Montgomery), infinity = all-zero limbs.  out may alias in.
int zk_g1_normalize(void* out, const void* in, size_t n, void* st) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_g1_normalize<false>, dim3(cdiv(cdiv(n, CH), GT)), dim3(GT), 0, (hipStream_t)st, out, (const G1Jac*)in, n);
    ZK_LAUNCH_CHECK();
    return 0;
}

// Commitment::commit_int (commitment.cu:50-58): out[row] = sum_j [t[row,j]] gens[j], t = embedded int32 values.
// scalars: Fr tensor of m*ngen elements.  Values outside the int32 embedding are rejected.
int zk_g1_commit_int(void* out, const void* gens, const void* scalars_fr, size_t m, size_t ngen, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (m == 0) return 0;
    ZK_ARG(ngen >= 1, "zk_g1_commit_int: no generators");
    ZK_ARG(m <= 0x7fffffffu, "zk_g1_commit_int: too many rows");
    const size_t total = m * ngen;
    Scratch ints(sizeof(int32_t) * total, st), flags(8, st);
    if (ints.rc) return ints.rc;
    if (flags.rc) return flags.rc;
    ZK_HIP(hipMemsetAsync(flags.p, 0, 8, st));
    hipLaunchKernelGGL(k_fr_to_i32_checked, dim3(cdiv(total, 256)), dim3(256), 0, st, ints.as<int32_t>(), flags.as<uint32_t>(), flags.as<uint32_t>() + 1, (const Fr*)scalars_fr, total);
    ZK_LAUNCH_CHECK();
    void* stage = nullptr;
    int rc = staging(&stage, 8);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, flags.p, 8, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    const uint32_t bad = ((uint32_t*)stage)[0], maxabs = ((uint32_t*)stage)[1];
    ZK_ARG(bad == 0, "zk_g1_commit_int: a scalar is not the embedding of an int32 value");
    // window width: wide tables pay off when many rows share the generators
    const uint32_t c = (m >= 256) ? 8u : (m >= 16 ? 5u : 3u);
    uint32_t bits = 0;
    while (bits < 32 && (maxabs >> bits)) ++bits;
    uint32_t nwin = (bits + 1 + c - 1) / c;   // one spare bit for the signed-digit carry
    if (nwin == 0) nwin = 1;
    const uint32_t half = 1u << (c - 1);
    const size_t tab_n = (size_t)nwin * ngen * half;
    Scratch tabj(sizeof(G1Jac) * tab_n, st), taba(sizeof(G1Affine) * tab_n, st);
    if (tabj.rc) return tabj.rc;
    if (taba.rc) return taba.rc;
    hipLaunchKernelGGL(k_msm_table_bases, dim3(cdiv(ngen, GT)), dim3(GT), 0, st, tabj.as<G1Jac>(), (const G1Jac*)gens, ngen, c, nwin);
    for (uint32_t logk = 0; logk + 1 < c; ++logk)
        hipLaunchKernelGGL(k_msm_table_fill, dim3(cdiv(((size_t)nwin * ngen) << logk, GT)), dim3(GT), 0, st, tabj.as<G1Jac>(), (size_t)nwin * ngen, c - 1, logk);
    hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(tab_n, CH), GT)), dim3(GT), 0, st, taba.p, tabj.as<G1Jac>(), tab_n);
    Scratch tab29(sizeof(A29) * tab_n, st);
    if (tab29.rc) return tab29.rc;
    hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(tab_n, 256)), dim3(256), 0, st, tab29.as<A29>(), taba.as<G1Affine>(), tab_n);
    ZK_LAUNCH_CHECK();
    uint32_t nseg = 1;
    if (m < 2048) { nseg = (uint32_t)(2048 / m); const uint32_t cap = (uint32_t)((ngen + GT - 1) / GT); if (nseg > cap) nseg = cap; if (nseg < 1) nseg = 1; }
    if (nseg == 1) {
        hipLaunchKernelGGL(k_msm_rows, dim3((unsigned)m, 1), dim3(GT), 0, st, (G1Jac*)out, tab29.as<A29>(), ints.as<int32_t>(), ngen, c, nwin, 1u);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    Scratch part(sizeof(G1Jac) * m * nseg, st);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_msm_rows, dim3((unsigned)m, nseg), dim3(GT), 0, st, part.as<G1Jac>(), tab29.as<A29>(), ints.as<int32_t>(), ngen, c, nwin, nseg);
    hipLaunchKernelGGL(k_g1_rowsum, dim3((unsigned)m, 1), dim3(GT), 0, st, (G1Jac*)out, part.as<G1Jac>(), (size_t)nseg, 1u);
    ZK_LAUNCH_CHECK();
    return 0;
}

// out[i] = [s_i] B for a base point B given on the host (Jacobian, Montgomery form) and n scalars in standard form: what
// Commitment::random does with the group generator (commitment.cu:3-8, a broadcast G1Jacobian_mul).  The table of B's
// multiples is kept on the device from one call to the next with the same base (one table per process, 4224 points).
int zk_g1_fixed_base_mul(void* out, const uint32_t* base_host, const void* scalars_fr, size_t n, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    if (n == 0) return 0;
    static std::mutex mu;
    static void* tab = nullptr;
    static int tab_dev = -1;
    static uint32_t tab_base[36];
    std::lock_guard<std::mutex> lk(mu);
    int dev = 0;
    ZK_HIP(hipGetDevice(&dev));
    if (!tab || tab_dev != dev || std::memcmp(tab_base, base_host, sizeof(tab_base)) != 0) {
        const size_t tab_n = (size_t)FB_WIN * 128;
        if (tab && tab_dev != dev) { int cur = dev; ZK_HIP(hipSetDevice(tab_dev)); ZK_HIP(hipFree(tab)); ZK_HIP(hipSetDevice(cur)); tab = nullptr; }
        if (!tab) ZK_HIP(hipMalloc(&tab, sizeof(A29) * tab_n));
        tab_dev = -1;                                   // not valid until the build below has finished
        Scratch b(sizeof(G1Jac), st), tabj(sizeof(G1Jac) * tab_n, st), taba(sizeof(G1Affine) * tab_n, st);
        if (b.rc) return b.rc;
        if (tabj.rc) return tabj.rc;
        if (taba.rc) return taba.rc;
        ZK_HIP(hipMemcpyAsync(b.p, base_host, sizeof(G1Jac), hipMemcpyHostToDevice, st));
        hipLaunchKernelGGL(k_msm_table_bases, dim3(1), dim3(GT), 0, st, tabj.as<G1Jac>(), b.as<G1Jac>(), (size_t)1, 8u, FB_WIN);
        for (uint32_t logk = 0; logk < 7; ++logk)
            hipLaunchKernelGGL(k_msm_table_fill, dim3(cdiv((size_t)FB_WIN << logk, GT)), dim3(GT), 0, st, tabj.as<G1Jac>(), (size_t)FB_WIN, 7u, logk);
        hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(tab_n, CH), GT)), dim3(GT), 0, st, taba.p, tabj.as<G1Jac>(), tab_n);
        hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(tab_n, 256)), dim3(256), 0, st, (A29*)tab, taba.as<G1Affine>(), tab_n);
        ZK_LAUNCH_CHECK();
        ZK_HIP(hipStreamSynchronize(st));               // later calls may come on other streams
        std::memcpy(tab_base, base_host, sizeof(tab_base));
        tab_dev = dev;
    }
    hipLaunchKernelGGL(k_g1_fixed_base_mul, dim3(cdiv(n, GT)), dim3(GT), 0, st, (G1Jac*)out, (const A29*)tab, (const Fr*)scalars_fr, n);
    ZK_LAUNCH_CHECK();
    return 0;
}

// One round of Commitment::me_open (commitment.cu:79-129) with all three sums computed directly.  u: standard-form
// challenge (the field scalar of the fold and the integer of the scalar multiplications, as in the reference).
// new_scalars / new_gens: (old_size+1)/2 elements.  sums_host: 3 points (T, T0, T1), normalised to z = 1.
int zk_g1_open_round(void* new_scalars, void* new_gens, uint32_t* sums_host, const void* scalars, const void* gens, const uint32_t* u, size_t old_size, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(old_size >= 1, "zk_g1_open_round: empty input");
    const size_t new_size = (old_size + 1) / 2;
    Scratch pts(sizeof(G1Jac) * 3, st);
    if (pts.rc) return pts.rc;
    Scratch wsum(sizeof(G1Jac) * 3 * MW, st);
    if (wsum.rc) return wsum.rc;
    Arena arena(st);
    Scratch& g29 = arena.add(sizeof(A29) * (old_size + new_size));
    Scratch& n29 = arena.add(sizeof(A29) * new_size);
    if (g29.rc || n29.rc) return g29.rc ? g29.rc : n29.rc;
    int rc = open_prep_build(g29.as<A29>(), (const G1Jac*)gens, old_size, arena, st);
    if (rc) return rc;
    std::vector<hipEvent_t> evs;
    const RoundItem item{(Fr*)new_scalars, n29.as<A29>(), (const Fr*)scalars, g29.as<A29>(), load_fr(u), nullptr};
    rc = open_round_launch(&item, 1, old_size, true, 0, wsum.as<G1Jac>(), 0u, arena, st, st, evs);
    (void)evs;
    if (rc) return rc;
    hipLaunchKernelGGL(k_a29_to_jac, dim3(cdiv(new_size, GT)), dim3(GT), 0, st, (G1Jac*)new_gens, n29.as<A29>(), new_size);
    hipLaunchKernelGGL(k_open_horner, dim3(3, 1), dim3(GT), 0, st, pts.as<G1Jac>(), wsum.as<G1Jac>(), 1u, 3u, 0u);
    hipLaunchKernelGGL(k_g1_normalize<false>, dim3(1), dim3(GT), 0, st, pts.p, pts.as<G1Jac>(), (size_t)3);
    ZK_LAUNCH_CHECK();
    void* stage = nullptr;
    rc = staging(&stage, sizeof(G1Jac) * 3);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, pts.p, sizeof(G1Jac) * 3, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    memcpy(sums_host, stage, sizeof(G1Jac) * 3);
    return 0;
}

// The whole recursion of Commitment::me_open (commitment.cu:109-129): `rounds` halvings of (scalars, gens) of length n
// with the challenges u[0..rounds).  An OpenJob queues all of it on one stream and keeps every buffer until the
// result has been fetched.
struct OpenJob {
    Arena arena;
    hipStream_t st = nullptr;
    int rounds = 0, count = 0;
    G1Jac* pts = nullptr;                      // count x (3 rounds + 1) points
    const Fr* final_scalar[OB_MAX] = {};
    hipEvent_t ready = nullptr;    // only for jobs on a side stream
    hipStream_t aux = nullptr;     // second stream of the job (bucket sums beside the folds); equals st when the job has one stream
    std::vector<hipEvent_t> events;
    void* pin = nullptr;           // pinned host buffer behind the job's challenges and descriptors
    void* pin2 = nullptr;          // and behind the list of its rounds' bucket reductions
    uint64_t ticket = 0;           // the launch thread's ticket while it queues the job's kernels
    int queue_rc = 0;              // what queuing returned, and its message
    std::string queue_err;
    ~OpenJob() { pinned_release(pin); pinned_release(pin2); }
};
// One opening of the batch: its scalars, its challenges (rounds x 8 limbs) and its generators -- Jacobian, or null when
// `prep` (their prepared form, open_prep_build) is given
struct OpenItem { const void* scalars; const void* gens; const A29* prep; const uint32_t* u; const A29* comb = nullptr; const A29* comb2 = nullptr;
                  const void* rows = nullptr; uint32_t nrows = 0; const uint32_t* u_rows = nullptr; int k_rows = 0; int cross_rounds = 0;
                  const A29* comb3 = nullptr; };
// The targets of every opening of a batch (T of round 0, then T0, T1 of the first `full` rounds) as bucket sums over the
// openings' [pattern][row] points, on aux.  The raw buckets' reductions are appended to `later`: the caller runs them with
// those of its halving rounds, so the 248 doublings of a reduction are waited for once per job.
static int open_cross_sums_queue(Arena& arena, const OpenItem* items, int count, int full, G1Jac* wsum, uint32_t wstride, const Fr* const* urow_dev, const Fr* U_dev, int rounds,
                                 hipStream_t aux, std::vector<PointDesc>& later) {
    const uint32_t ntargets = 1u + 2u * (uint32_t)full;
    const uint32_t npatterns = 1u + 2u * (((1u << (2 * full)) - 1u) / 3u);
    const uint32_t widest = full ? (1u << (2 * (full - 1))) : 1u;           // patterns of the largest target
    CrossDigitBatch db;
    const A29* base[OB_MAX];
    const int8_t* digs[OB_MAX];
    size_t most_terms = 0, most_count = 0;
    for (int i = 0; i < count; ++i) {
        const size_t terms = (size_t)npatterns * items[i].nrows;
        ZK_ARG(items[i].nrows >= 1 && terms < (1ull << 31), "zk_g1_open: bad row count");
        most_terms = std::max(most_terms, terms);
        most_count = std::max(most_count, (size_t)widest * items[i].nrows);
        Scratch& aff = arena.add(sizeof(G1Affine) * terms);
        Scratch& a29 = arena.add(sizeof(A29) * terms);
        Scratch& dg = arena.add((size_t)(MW + 1) * terms);
        if (aff.rc || a29.rc || dg.rc) return aff.rc ? aff.rc : (a29.rc ? a29.rc : dg.rc);
        hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(terms, CH), GT)), dim3(GT), 0, aux, aff.p, (const G1Jac*)items[i].rows, terms);
        hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(terms, 256)), dim3(256), 0, aux, a29.as<A29>(), aff.as<G1Affine>(), terms);
        base[i] = a29.as<A29>();
        digs[i] = dg.as<int8_t>();
        db.it[i] = CrossDigitItem{dg.as<int8_t>(), urow_dev[i], U_dev + (size_t)i * rounds, items[i].nrows, (uint32_t)items[i].k_rows};
    }
    for (int i = count; i < OB_MAX; ++i) db.it[i] = db.it[0];
    hipLaunchKernelGGL(k_open_cross_digits, dim3(cdiv(most_terms, 256), count), dim3(256), 0, aux, db, npatterns);
    ZK_LAUNCH_CHECK();
    const uint32_t chunks = cdiv(most_count, MSEG);
    const uint32_t cps = (chunks + 255u) / 256u;
    const uint32_t nseg = (chunks + cps - 1) / cps;
    const uint32_t n_msm = ntargets * (uint32_t)count;
    Scratch& partial = arena.add(sizeof(G1Jac) * n_msm * MW * (size_t)nseg * MT);
    if (partial.rc) return partial.rc;
    const int per = std::max(1, OB_SUMS / (int)ntargets);                  // openings whose targets fit one launch's descriptors
    for (int g0 = 0; g0 < count; g0 += per) {
        const int gc = std::min(per, count - g0);
        MsmDescs<OB_SUMS> descs;
        uint32_t z = 0;
        for (int i = g0; i < g0 + gc; ++i)
            for (uint32_t t = 0; t < ntargets; ++t) {
                uint32_t q, p0, npat, slot;
                cross_target(t, q, p0, npat, slot);
                const uint32_t terms = npatterns * items[i].nrows, off = p0 * items[i].nrows;
                descs.d[z++] = MsmDesc{digs[i], base[i], terms, npat * items[i].nrows, 1u, off, 1u, off, 0u};
            }
        const uint32_t used = z;
        for (; z < (uint32_t)OB_SUMS; ++z) descs.d[z] = MsmDesc{digs[0], base[0], 0u, 0u, 1u, 0u, 1u, 0u, 0u};
        hipLaunchKernelGGL(k_msm_seg<OB_SUMS>, dim3(nseg, MW, used), dim3(MSL), 0, aux, partial.as<G1Jac>() + (size_t)g0 * ntargets * MW * nseg * MT, descs, (const MsmDesc*)nullptr,
                           nseg, cps);
    }
    const G1Jac* cur = partial.as<G1Jac>();
    uint32_t ns = nseg;
    while (ns > 1) {
        const uint32_t ng = (ns + 7) / 8;
        Scratch& nxt = arena.add(sizeof(G1Jac) * n_msm * MW * (size_t)ng * MT);
        if (nxt.rc) return nxt.rc;
        hipLaunchKernelGGL(k_msm_bucket_fold, dim3(n_msm * MW, ng), dim3(MT), 0, aux, nxt.as<G1Jac>(), cur, ns);
        cur = nxt.as<G1Jac>();
        ns = ng;
    }
    ZK_LAUNCH_CHECK();
    for (int i = 0; i < count; ++i)
        for (uint32_t t = 0; t < ntargets; ++t) {
            uint32_t q, p0, npat, slot;
            cross_target(t, q, p0, npat, slot);
            later.push_back(PointDesc{cur + ((size_t)i * ntargets + t) * MW * ns * MT, wsum + (size_t)wstride * i + slot, ns, 0u});
        }
    return 0;
}
// rows (optional): commitments of the opened tensor's rows, [pattern][row] as open_cross_sums_queue takes them -- the row
// commitments alone (cross_rounds = 0) or with the cross patterns of the first cross_rounds rounds
static int open_queue(OpenJob& job, const OpenItem* items, int count, size_t n, int rounds, hipStream_t st, hipStream_t aux) {
    ZK_ARG(n >= 1, "zk_g1_open: empty input");
    ZK_ARG(count >= 1 && count <= OB_MAX, "zk_g1_open: a batch holds 1 to 8 openings");
    ZK_ARG(rounds >= 0 && rounds <= 64, "zk_g1_open: bad round count");
    ZK_ARG(sizeof(G1Jac) * (3 * (size_t)rounds + 1) + sizeof(Fr) <= 65536, "zk_g1_open: proof larger than the staging buffer");
    job.st = st;
    job.aux = aux;
    job.arena.streams(st, aux);      // blocks serve kernels of both streams; aux joins st before the job ends
    job.rounds = rounds;
    job.count = count;
    const size_t npts = 3 * (size_t)rounds + 1;
    const uint32_t wstride = 3u * MW * (uint32_t)(rounds ? rounds : 1);      // window sums of one opening's halving rounds
    Scratch& pts = job.arena.add(sizeof(G1Jac) * npts * count);
    Scratch& wsum = job.arena.add(sizeof(G1Jac) * (size_t)wstride * count);
    if (pts.rc) return pts.rc;
    if (wsum.rc) return wsum.rc;
    job.pts = pts.as<G1Jac>();
    size_t n_urows = 0;
    for (int i = 0; i < count; ++i) n_urows += items[i].rows ? (size_t)items[i].k_rows : 0;
    ZK_ARG(sizeof(Fr) * ((size_t)rounds * count + n_urows) <= JOB_U_BYTES, "zk_g1_open: too many rounds for the batch");
    Scratch& jdev = job.arena.add(JOB_U_BYTES + JOB_DESC_BYTES);
    if (jdev.rc) return jdev.rc;
    {
        int prc = pinned_acquire(&job.pin);
        if (prc) return prc;
        Fr* hu = (Fr*)job.pin;
        for (int i = 0; i < count; ++i)
            for (int r = 0; r < rounds; ++r) hu[(size_t)i * rounds + r] = to_mont(load_fr(items[i].u + 8 * r));
        size_t at = (size_t)rounds * count;           // the row challenges follow
        for (int i = 0; i < count; ++i)
            if (items[i].rows)
                for (int j = 0; j < items[i].k_rows; ++j) hu[at++] = to_mont(load_fr(items[i].u_rows + 8 * j));
        if (at) ZK_HIP(hipMemcpyAsync(jdev.p, job.pin, sizeof(Fr) * at, hipMemcpyHostToDevice, st));
    }
    const Fr* U_dev = jdev.as<Fr>();
    const Fr* urow_dev[OB_MAX];
    {
        size_t at = (size_t)rounds * count;
        for (int i = 0; i < count; ++i) { urow_dev[i] = U_dev + at; if (items[i].rows) at += (size_t)items[i].k_rows; }
    }
    const Fr* cs[OB_MAX];
    const A29* cg[OB_MAX];
    for (int i = 0; i < count; ++i) {
        cs[i] = (const Fr*)items[i].scalars;
        cg[i] = items[i].prep;
        if (!cg[i]) {
            Scratch& g29 = job.arena.add(sizeof(A29) * (n + (n + 1) / 2));
            if (g29.rc) return g29.rc;
            int rc = open_prep_build(g29.as<A29>(), (const G1Jac*)items[i].gens, n, job.arena, st);
            if (rc) return rc;
            cg[i] = g29.as<A29>();
        }
    }
    // commitments of the tensors' rows: which sums they replace (all openings of the batch must bring them)
    bool with_rows = true;
    int cross_r = 64;
    for (int i = 0; i < count; ++i) { with_rows = with_rows && items[i].rows != nullptr; cross_r = std::min(cross_r, items[i].cross_rounds); }
    if (!with_rows) cross_r = 0;
    int rounds_from_rows = 0;                 // halving rounds that take sums from the row commitments
    if (with_rows) {
        int halving = 0;
        size_t sz = n;
        for (int r = 0; r < rounds && !(sz <= (size_t)TAIL_N && rounds - r <= TAIL_LEVELS); ++r) { ++halving; sz = (sz + 1) / 2; }
        rounds_from_rows = std::min(halving, std::max(cross_r, 1));
    }
    std::vector<PointDesc> later;        // bucket reductions that nothing waits for before the end: one launch behind the last round
    if (rounds_from_rows > 0) {
        if (aux != st) {          // the challenges travel on st
            hipEvent_t up;
            ZK_HIP(hipEventCreateWithFlags(&up, hipEventDisableTiming));
            job.events.push_back(up);
            ZK_HIP(hipEventRecord(up, st));
            ZK_HIP(hipStreamWaitEvent(aux, up, 0));
        }
        int rc = open_cross_sums_queue(job.arena, items, count, std::min(rounds_from_rows, cross_r), wsum.as<G1Jac>(), wstride, urow_dev, U_dev, rounds, aux, later);
        if (rc) return rc;
    }
    size_t size = n;
    int halving_rounds = rounds;
    bool tail_done = false;
    int r_first = 0;
    // three rounds as one fold: every opening brings the jump tables and cross commitments for those rounds, and all
    // three are halving rounds
    {
        bool jump = with_rows && cross_r >= JUMP_ROUNDS && rounds_from_rows >= JUMP_ROUNDS && rounds >= JUMP_ROUNDS && !(n & (n - 1));
        for (int i = 0; i < count; ++i) jump = jump && items[i].comb3 != nullptr;
        if (jump) {
            const size_t ns = n >> JUMP_ROUNDS;
            Scratch& s2 = job.arena.add(sizeof(Fr) * ns * count);
            Scratch& g2 = job.arena.add(sizeof(A29) * ns * count);
            if (s2.rc) return s2.rc;
            if (g2.rc) return g2.rc;
            JumpBatch jb;
            double fp_mults = 0;
            const Fr one = big_one_mont<8>();
            for (int i = 0; i < OB_MAX; ++i) {
                const int k = i < count ? i : 0;
                JumpItem& f = jb.it[i];
                f.ns = s2.as<Fr>() + ns * k; f.ng = g2.as<A29>() + ns * k; f.s = cs[k]; f.g = cg[k]; f.tab = items[k].comb3;
                Fr um[JUMP_ROUNDS];
                for (int q = 0; q < JUMP_ROUNDS; ++q) um[q] = f.u_mont[q] = to_mont(load_fr(items[k].u + 8 * q));
                for (int b = 0; b < JUMP_TABS; ++b) {
                    Fr c = one;           // c_b = prod_q (bit_q(b) ? 1 - u_q : u_q)
                    for (int q = 0; q < JUMP_ROUNDS; ++q) c = mont_mul(c, ((b >> q) & 1) ? sub(one, um[q]) : um[q]);
                    f.ck[b] = comb_of(glv_split(from_mont(c)));
                    if (i < count) fp_mults += (comb_fp_mults_per_pair(f.ck[b]) - 7.0 * COMB_W - 19.0) * (double)ns;
                }
                if (i < count) fp_mults += (7.0 * COMB_W + 19.0) * (double)ns;
            }
            hipEvent_t t0 = nullptr, t1 = nullptr;
            if (g_fold_timer.on) {
                ZK_HIP(hipEventCreate(&t0));
                ZK_HIP(hipEventCreate(&t1));
                ZK_HIP(hipEventRecord(t0, st));
            }
            hipLaunchKernelGGL(k_open_fold_jump, dim3(cdiv(ns, GT), count), dim3(GT), 0, st, jb, ns);
            ZK_LAUNCH_CHECK();
            if (g_fold_timer.on) {
                ZK_HIP(hipEventRecord(t1, st));
                std::lock_guard<std::mutex> lk(g_fold_timer.mu);
                g_fold_timer.ev.emplace_back(t0, t1);
                g_fold_timer.fp_mults += fp_mults;
                g_fold_timer.pairs += ns * (size_t)count * (JUMP_SPAN - 1);       // pairs the three rounds fold: 4 + 2 + 1 per result
                g_fold_timer.method.push_back(2);
                g_fold_timer.m_mults[2] += fp_mults;
                g_fold_timer.m_pairs[2] += ns * (size_t)count * (JUMP_SPAN - 1);
            }
            for (int i = 0; i < count; ++i) { cs[i] = s2.as<Fr>() + ns * i; cg[i] = g2.as<A29>() + ns * i; }
            size = ns;
            r_first = JUMP_ROUNDS;
        }
    }
    for (int r = r_first; r < rounds; ++r) {
        if (size <= (size_t)TAIL_N && rounds - r <= TAIL_LEVELS) {
            int rc = open_tail_launch(cs, cg, count, size, rounds - r, r, rounds, pts.as<G1Jac>(), U_dev, job.pin, (char*)jdev.p + JOB_U_BYTES, job.arena, st);
            if (rc) return rc;
            halving_rounds = r;
            tail_done = true;
            break;
        }
        const size_t ns = (size + 1) / 2;
        Scratch& s2 = job.arena.add(sizeof(Fr) * ns * count);
        Scratch& g2 = job.arena.add(sizeof(A29) * ns * count);
        if (s2.rc) return s2.rc;
        if (g2.rc) return g2.rc;
        RoundItem ri[OB_MAX];
        for (int i = 0; i < count; ++i) {
            ri[i] = RoundItem{s2.as<Fr>() + ns * i, g2.as<A29>() + ns * i, cs[i], cg[i], load_fr(items[i].u + 8 * r)};
            if (r == 0) ri[i].comb = items[i].comb;
            if (r == 1) { ri[i].comb2 = items[i].comb2; ri[i].u_prev = load_fr(items[i].u + 8 * (r - 1)); }
        }
        const int given = !with_rows ? 0 : (r < cross_r ? 2 : (r == 0 ? 1 : 0));
        int rc = open_round_launch(ri, count, size, r == 0, given, wsum.as<G1Jac>() + (size_t)3 * MW * r, wstride, job.arena, st, aux, job.events, aux != st ? &later : nullptr);
        if (rc) return rc;
        for (int i = 0; i < count; ++i) { cs[i] = ri[i].new_scalars; cg[i] = ri[i].new_gens; }
        size = ns;
    }
    if (!later.empty()) {
        ZK_ARG(sizeof(PointDesc) * later.size() <= 65536, "zk_g1_open: too many sums");
        int prc = pinned_acquire(&job.pin2);
        if (prc) return prc;
        memcpy(job.pin2, later.data(), sizeof(PointDesc) * later.size());
        Scratch& ld = job.arena.add(sizeof(PointDesc) * later.size());
        if (ld.rc) return ld.rc;
        ZK_HIP(hipMemcpyAsync(ld.p, job.pin2, sizeof(PointDesc) * later.size(), hipMemcpyHostToDevice, aux));
        hipLaunchKernelGGL(k_msm_point, dim3((unsigned)later.size()), dim3(MT), 0, aux, (G1Jac*)nullptr, (G1Jac*)nullptr, (const MsmDesc*)nullptr, (const G1Jac*)nullptr, 0u, 1u, 0u,
                           (const PointDesc*)ld.p);
        ZK_LAUNCH_CHECK();
    }
    // the single points of the halving rounds, behind the last bucket sums
    if (halving_rounds > 0) {
        hipLaunchKernelGGL(k_open_horner, dim3(3 * halving_rounds, count), dim3(GT), 0, aux, pts.as<G1Jac>(), wsum.as<G1Jac>(), (uint32_t)halving_rounds, (uint32_t)npts, wstride);
        if (halving_rounds > 1)
            hipLaunchKernelGGL(k_open_chain, dim3(halving_rounds - 1, count), dim3(GT), 0, aux, pts.as<G1Jac>(), U_dev, (uint32_t)halving_rounds, (uint32_t)npts, (uint32_t)rounds);
        ZK_LAUNCH_CHECK();
    }
    if (aux != st) {
        hipEvent_t done;
        ZK_HIP(hipEventCreateWithFlags(&done, hipEventDisableTiming));
        job.events.push_back(done);
        ZK_HIP(hipEventRecord(done, aux));
        ZK_HIP(hipStreamWaitEvent(st, done, 0));
    }
    if (!tail_done)
        for (int i = 0; i < count; ++i) hipLaunchKernelGGL(k_open_finish, dim3(1), dim3(GT), 0, st, pts.as<G1Jac>() + npts * i, cg[i], (uint32_t)rounds);
    hipLaunchKernelGGL(k_g1_normalize<false>, dim3(cdiv(cdiv(npts * count, CH), GT)), dim3(GT), 0, st, pts.p, pts.as<G1Jac>(), npts * count);
    ZK_LAUNCH_CHECK();
    for (int i = 0; i < count; ++i) job.final_scalar[i] = cs[i];
    return 0;
}
// waits for the job's stream and copies the proof points and the folded scalars out: opening i's points at
// proof_host + i * (3 rounds + 1) * 36, its scalar at final_scalar_host + i * 8
static int open_collect(OpenJob& job, uint32_t* proof_host, uint32_t* final_scalar_host) {
    const size_t npts = 3 * (size_t)job.rounds + 1;
    void* stage = nullptr;
    int rc = staging(&stage, sizeof(G1Jac) * npts + sizeof(Fr));
    if (rc) return rc;
    for (int i = 0; i < job.count; ++i) {
        ZK_HIP(hipMemcpyAsync(stage, job.pts + npts * i, sizeof(G1Jac) * npts, hipMemcpyDeviceToHost, job.st));
        ZK_HIP(hipMemcpyAsync((char*)stage + sizeof(G1Jac) * npts, job.final_scalar[i], sizeof(Fr), hipMemcpyDeviceToHost, job.st));
        ZK_HIP(hipStreamSynchronize(job.st));
        memcpy(proof_host + 36 * npts * i, stage, sizeof(G1Jac) * npts);
        memcpy(final_scalar_host + 8 * (size_t)i, (char*)stage + sizeof(G1Jac) * npts, sizeof(Fr));
    }
    return 0;
}
// proof_host receives 3*rounds + 1 points: T, T0, T1 of every round, then the folded generator; all normalised to
// z = 1 (infinity: all-zero limbs).  final_scalar_host: the folded scalar.
int zk_g1_open(uint32_t* proof_host, uint32_t* final_scalar_host, const void* scalars, const void* gens, size_t n, const uint32_t* u, int rounds, void* stv) {
    OpenJob job;
    const OpenItem item{scalars, gens, nullptr, u};
    int rc = open_queue(job, &item, 1, n, rounds, (hipStream_t)stv, (hipStream_t)stv);
    if (rc) { (void)hipStreamSynchronize((hipStream_t)stv); return rc; }
    return open_collect(job, proof_host, final_scalar_host);
}
// The same in two halves.  begin queues the recursion on a stream of the library's own, ordered after everything queued
// on `stream` so far, and returns at once; the caller goes on using `stream`, and both run side by side.  scalars and gens
// must stay alive and unmodified until end, which waits for the opening, delivers its results and releases its buffers.
static int open_begin_impl(void** handle, const OpenItem* items, int count, size_t n, int rounds, void* stv) {
    ZK_ARG(handle != nullptr, "zk_g1_open_begin: null handle");
    hipStream_t side = side_stream(0), aux = side_stream(0);      // consecutive streams of the pool: the folds on one, the bucket sums on the other
    ZK_ARG(side != nullptr && aux != nullptr, "zk_g1_open_begin: could not create a stream");
    // what open_queue refuses is refused here, before anything is handed to the launch thread
    ZK_ARG(n >= 1, "zk_g1_open: empty input");
    ZK_ARG(count >= 1 && count <= OB_MAX, "zk_g1_open: a batch holds 1 to 8 openings");
    ZK_ARG(rounds >= 0 && rounds <= 64, "zk_g1_open: bad round count");
    ZK_ARG(sizeof(G1Jac) * (3 * (size_t)rounds + 1) + sizeof(Fr) <= 65536, "zk_g1_open: proof larger than the staging buffer");
    std::unique_ptr<OpenJob> job(new OpenJob);
    ZK_HIP(hipEventCreateWithFlags(&job->ready, hipEventDisableTiming));
    ZK_HIP(hipEventRecord(job->ready, (hipStream_t)stv));
    ZK_HIP(hipStreamWaitEvent(side, job->ready, 0));
    pool_note_wait((hipStream_t)stv, side);
    if (!launcher_enabled()) {
        int rc = open_queue(*job, items, count, n, rounds, side, aux);
        if (rc) {
            (void)hipStreamSynchronize(side);
            (void)hipStreamSynchronize(aux);
            for (hipEvent_t e : job->events) (void)hipEventDestroy(e);
            (void)hipEventDestroy(job->ready);
            return rc;
        }
        *handle = job.release();
        return 0;
    }
    // The launch thread queues the job's few hundred launches (a millisecond of host time an opening) while the caller
    // goes on; zk_g1_open_end waits for the ticket and reports what queuing returned.  The challenge arrays are the
    // caller's and only valid during this call: the job takes copies.
    struct Owned { OpenItem items[OB_MAX]; std::vector<uint32_t> u[OB_MAX], u_rows[OB_MAX]; };
    std::shared_ptr<Owned> own(new Owned);
    for (int i = 0; i < count; ++i) {
        own->items[i] = items[i];
        own->u[i].assign(items[i].u, items[i].u + 8 * (size_t)rounds);
        own->items[i].u = own->u[i].data();
        if (items[i].rows && items[i].k_rows > 0) {
            own->u_rows[i].assign(items[i].u_rows, items[i].u_rows + 8 * (size_t)items[i].k_rows);
            own->items[i].u_rows = own->u_rows[i].data();
        }
    }
    OpenJob* j = job.get();
    j->st = side;
    j->aux = aux;
    j->ticket = launcher_submit([j, own, count, n, rounds, side, aux] {
        j->queue_rc = open_queue(*j, own->items, count, n, rounds, side, aux);
        if (j->queue_rc) j->queue_err = last_error_text();
    });
    *handle = job.release();
    return 0;
}
int zk_g1_open_begin(void** handle, const void* scalars, const void* gens, size_t n, const uint32_t* u, int rounds, void* stv) {
    const OpenItem item{scalars, gens, nullptr, u};
    return open_begin_impl(handle, &item, 1, n, rounds, stv);
}
// Generators prepared once for any number of openings against them: their affine 29-bit-limb form and the pair sums of
// the first round (weight-independent; 1.5 n points of 112 bytes).  The handle is freed with zk_g1_open_prepared_free
// once no opening that uses it is pending.
struct OpenPrepared { void* a29 = nullptr; size_t n = 0; void* comb = nullptr; void* comb2 = nullptr; void* comb3 = nullptr; size_t table_bytes = 0; };      // comb3: k_open_fold_jump's tables (instead of the other two)
static int open_prepare_impl(void** prepared, const void* gens, size_t n, int table_mode, void* stv);
int zk_g1_open_prepare(void** prepared, const void* gens, size_t n, void* stv) { return open_prepare_impl(prepared, gens, n, 2, stv); }
int zk_g1_open_prepare_tables(void** prepared, const void* gens, size_t n, int tables, void* stv) {
    ZK_ARG(tables >= 0 && tables <= 3, "zk_g1_open_prepare_tables: tables 0 to 3");
    return open_prepare_impl(prepared, gens, n, tables, stv);
}
// bytes of fold tables that zk_g1_open_prepare_tables(.., tables) keeps for n generators (0 where that mode makes none for this n)
static size_t open_table_bytes(size_t n, int tables) {
    if (tables >= 3 && !(n & (n - 1)) && (n >> JUMP_ROUNDS) >= (size_t)TAIL_N) return sizeof(A29) * (n >> JUMP_ROUNDS) * COMB_N * JUMP_TABS;
    if (tables < 1 || n <= (size_t)TAIL_N) return 0;
    const size_t np = (n + 1) / 2, nq = (np + 1) / 2;
    size_t b = sizeof(A29) * np * COMB_N;
    if (tables >= 2 && np > (size_t)TAIL_N) b += sizeof(A29) * 2 * nq * COMB_N;
    return b;
}
size_t zk_g1_open_table_bytes(size_t n, int tables) { return open_table_bytes(n, tables < 0 ? 0 : (tables > 3 ? 3 : tables)); }
// The richest tables that fit `max_table_bytes`: mode `want` (0..3) if its tables fit, else the next smaller mode, down to none.
int zk_g1_open_prepare_budget(void** prepared, const void* gens, size_t n, int want, size_t max_table_bytes, int* tables_made, void* stv) {
    ZK_ARG(want >= 0 && want <= 3, "zk_g1_open_prepare_budget: tables 0 to 3");
    int mode = want;
    while (mode > 0 && open_table_bytes(n, mode) > max_table_bytes) --mode;
    if (tables_made) *tables_made = mode;
    return open_prepare_impl(prepared, gens, n, mode, stv);
}
size_t zk_g1_open_prepared_table_bytes(const void* prepared) { return prepared ? ((const OpenPrepared*)prepared)->table_bytes : 0; }
static int open_prepare_impl(void** prepared, const void* gens, size_t n, int table_mode, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(prepared != nullptr && n >= 1, "zk_g1_open_prepare: null handle or no generators");
    std::unique_ptr<OpenPrepared> pr(new OpenPrepared);
    int rc = pool_alloc(&pr->a29, sizeof(A29) * (n + (n + 1) / 2), st);
    if (rc) return rc;
    pr->n = n;
    {
        Arena arena(st);
        rc = open_prep_build((A29*)pr->a29, (const G1Jac*)gens, n, arena, st);
        // The combs of the first two rounds, for each round that is a fold (more generators than the batched last rounds
        // take): entry-major tables of the subset sums of 2^(j COMB_W) P over the round's prepared points P (the pair
        // differences D; for the second round F and H, see k_open_fold_comb), built from elementwise point kernels -- the
        // teeth by repeated doubling (an addition of an array to itself), entry m = entry (m without its lowest bit) + entry
        // (that bit).
        // The tables only make the folds cheaper: ZKLLM_OPEN_TABLES = 0 or 1 keeps none or the first round's alone (28 KB
        // per generator pair and round), and when the device has no room for them or for their construction the handle
        // is made without them -- those rounds then walk (k_open_fold29), the results are the same.
        static const int env_rounds = [] { const char* e = getenv("ZKLLM_OPEN_TABLES"); return e ? atoi(e) : -1; }();
        const int table_rounds = env_rounds >= 0 ? env_rounds : table_mode;
        // mode 3: the seven tables of k_open_fold_jump in place of those two (as large as both together); only for a power of
        // two of generators that leaves more than the batched last rounds take after three folds
        const bool jump = table_rounds >= 3 && !(n & (n - 1)) && (n >> JUMP_ROUNDS) >= (size_t)TAIL_N;
        if (rc == 0 && jump) {
            const size_t no = n >> JUMP_ROUNDS, ne = no * COMB_N * JUMP_TABS;
            int trc = pool_alloc(&pr->comb3, sizeof(A29) * ne, st);
            Scratch& aff = arena.add(sizeof(G1Affine) * n);
            Scratch& tj = arena.add(sizeof(G1Jac) * ne);
            Scratch& ta = arena.add(sizeof(G1Affine) * ne);
            Scratch& tmp = arena.add(sizeof(G1Jac) * no);
            if (trc == 0) trc = aff.rc ? aff.rc : (tj.rc ? tj.rc : (ta.rc ? ta.rc : tmp.rc));
            if (trc) {
                if (pr->comb3) (void)pool_free(pr->comb3, st, true);
                pr->comb3 = nullptr;
            } else {
                static_assert(COMB_W % 2 == 0, "the doublings alternate between two buffers and must end in the table");
                hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(n, CH), GT)), dim3(GT), 0, st, aff.p, (const G1Jac*)gens, n);
                for (int b = 0; b < JUMP_TABS; ++b) {
                    G1Jac* T = tj.as<G1Jac>() + (size_t)b * COMB_N * no;
                    auto entry = [&](int m) { return T + (size_t)(m - 1) * no; };
                    hipLaunchKernelGGL(k_open_span_diff, dim3(cdiv(no, GT)), dim3(GT), 0, st, T, aff.as<G1Affine>(), (uint32_t)JUMP_SPAN, (uint32_t)b, no);
                    for (int t = 1; t < COMB_A; ++t) {
                        const G1Jac* src = entry(1 << (t - 1));
                        for (int k = 0; k < COMB_W; ++k) {          // no launch writes what it reads
                            G1Jac* dst = (k & 1) ? entry(1 << t) : tmp.as<G1Jac>();
                            hipLaunchKernelGGL(k_g1_add, dim3(cdiv(no, GT)), dim3(GT), 0, st, dst, src, src, no, no, 0);
                            src = dst;
                        }
                    }
                    for (int m = 3; m <= COMB_N; ++m) {
                        const int prev = m & (m - 1);
                        if (!prev) continue;
                        hipLaunchKernelGGL(k_g1_add, dim3(cdiv(no, GT)), dim3(GT), 0, st, entry(m), entry(prev), entry(m ^ prev), no, no, 0);
                    }
                }
                hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(ne, CH), GT)), dim3(GT), 0, st, ta.p, tj.as<G1Jac>(), ne);
                hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(ne, 256)), dim3(256), 0, st, (A29*)pr->comb3, ta.as<G1Affine>(), ne);
                if (hipGetLastError() != hipSuccess) rc = hip_fail(hipErrorLaunchFailure, "jump table build", __FILE__, __LINE__);
            }
        }
        if (rc == 0 && n > (size_t)TAIL_N && table_rounds >= 1 && !pr->comb3) {
            const size_t np = (n + 1) / 2, ne = np * COMB_N;
            const size_t nq = (np + 1) / 2, ne2 = nq * COMB_N;        // second round: two tables over the pairs of pairs
            bool second = np > (size_t)TAIL_N && table_rounds >= 2;   // that round is a fold too
            int trc = pool_alloc(&pr->comb, sizeof(A29) * ne, st);
            if (trc == 0 && second && pool_alloc(&pr->comb2, sizeof(A29) * 2 * ne2, st) != 0) { pr->comb2 = nullptr; second = false; }
            const size_t nt = second ? std::max(ne, 2 * ne2) : ne;
            Scratch& aff = arena.add(sizeof(G1Affine) * n);
            Scratch& tj = arena.add(sizeof(G1Jac) * nt);
            Scratch& ta = arena.add(sizeof(G1Affine) * nt);
            Scratch& tmp = arena.add(sizeof(G1Jac) * np);
            if (trc == 0) trc = aff.rc ? aff.rc : (tj.rc ? tj.rc : (ta.rc ? ta.rc : tmp.rc));
            if (trc) {                                                // nothing has been queued on the tables yet
                if (pr->comb) (void)pool_free(pr->comb, st, true);
                if (pr->comb2) (void)pool_free(pr->comb2, st, true);
                pr->comb = pr->comb2 = nullptr;
            } else {
                static_assert(COMB_W % 2 == 0, "the doublings alternate between two buffers and must end in the table");
                // T[0 .. cnt) holds entry 1 (the points themselves); fills the other COMB_N - 1 entries, cnt points each
                auto fill = [&](G1Jac* T, size_t cnt) {
                    auto entry = [&](int m) { return T + (size_t)(m - 1) * cnt; };
                    for (int t = 1; t < COMB_A; ++t) {
                        const G1Jac* src = entry(1 << (t - 1));
                        for (int k = 0; k < COMB_W; ++k) {          // no launch writes what it reads
                            G1Jac* dst = (k & 1) ? entry(1 << t) : tmp.as<G1Jac>();
                            hipLaunchKernelGGL(k_g1_add, dim3(cdiv(cnt, GT)), dim3(GT), 0, st, dst, src, src, cnt, cnt, 0);
                            src = dst;
                        }
                    }
                    for (int m = 3; m <= COMB_N; ++m) {
                        const int prev = m & (m - 1);
                        if (!prev) continue;
                        hipLaunchKernelGGL(k_g1_add, dim3(cdiv(cnt, GT)), dim3(GT), 0, st, entry(m), entry(prev), entry(m ^ prev), cnt, cnt, 0);
                    }
                };
                G1Jac* T = tj.as<G1Jac>();
                hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(n, CH), GT)), dim3(GT), 0, st, aff.p, (const G1Jac*)gens, n);
                hipLaunchKernelGGL(k_open_pair_points, dim3(cdiv(np, GT)), dim3(GT), 0, st, T, aff.as<G1Affine>(), n, np, 1);
                fill(T, np);
                hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(ne, CH), GT)), dim3(GT), 0, st, ta.p, tj.as<G1Jac>(), ne);
                hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(ne, 256)), dim3(256), 0, st, (A29*)pr->comb, ta.as<G1Affine>(), ne);
                if (second) {
                    // F from the odd-numbered generators, H from the first round's differences (entry 1 of its table, affine in ta);
                    // both are read before the buffers they sit in are written again
                    hipLaunchKernelGGL(k_open_pair_diff, dim3(cdiv(nq, GT)), dim3(GT), 0, st, T, aff.as<G1Affine>(), (size_t)1, (size_t)2, n / 2, nq);
                    hipLaunchKernelGGL(k_open_pair_diff, dim3(cdiv(nq, GT)), dim3(GT), 0, st, T + ne2, ta.as<G1Affine>(), (size_t)0, (size_t)1, np, nq);
                    fill(T, nq);
                    fill(T + ne2, nq);
                    hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(2 * ne2, CH), GT)), dim3(GT), 0, st, ta.p, tj.as<G1Jac>(), 2 * ne2);
                    hipLaunchKernelGGL(k_g1aff_to_a29, dim3(cdiv(2 * ne2, 256)), dim3(256), 0, st, (A29*)pr->comb2, ta.as<G1Affine>(), 2 * ne2);
                }
                if (rc == 0 && hipGetLastError() != hipSuccess) rc = hip_fail(hipErrorLaunchFailure, "comb build", __FILE__, __LINE__);
            }
        }
        // the temporaries go back to the allocator only when the stream has drained
        if (hipStreamSynchronize(st) != hipSuccess && rc == 0) rc = hip_fail(hipGetLastError(), "zk_g1_open_prepare sync", __FILE__, __LINE__);
        arena.mark_idle();
    }
    // (openings read the prepared form on the library's own streams: it is complete before the handle is handed out)
    if (rc) {
        (void)hipStreamSynchronize(st);
        pool_free(pr->a29, st, true);
        if (pr->comb) pool_free(pr->comb, st, true);
        if (pr->comb2) pool_free(pr->comb2, st, true);
        if (pr->comb3) pool_free(pr->comb3, st, true);
        return rc;
    }
    if (pr->comb3) pr->table_bytes += sizeof(A29) * (n >> JUMP_ROUNDS) * COMB_N * JUMP_TABS;
    if (pr->comb) pr->table_bytes += sizeof(A29) * ((n + 1) / 2) * COMB_N;
    if (pr->comb2) pr->table_bytes += sizeof(A29) * 2 * (((n + 1) / 2 + 1) / 2) * COMB_N;
    *prepared = pr.release();
    return 0;
}
int zk_g1_open_prepared_free(void* prepared) {
    if (!prepared) return 0;
    OpenPrepared* pr = (OpenPrepared*)prepared;
    int rc = pool_free(pr->a29, nullptr);
    if (pr->comb) (void)pool_free(pr->comb, nullptr);
    if (pr->comb2) (void)pool_free(pr->comb2, nullptr);
    if (pr->comb3) (void)pool_free(pr->comb3, nullptr);
    delete pr;
    return rc;
}
int zk_g1_open_begin_prepared(void** handle, const void* scalars, const void* prepared, const uint32_t* u, int rounds, void* stv) {
    ZK_ARG(prepared != nullptr, "zk_g1_open_begin_prepared: null generators");
    const OpenPrepared* pr = (const OpenPrepared*)prepared;
    OpenItem item{scalars, nullptr, (const A29*)pr->a29, u, (const A29*)pr->comb, (const A29*)pr->comb2};
    item.comb3 = (const A29*)pr->comb3;
    return open_begin_impl(handle, &item, 1, pr->n, rounds, stv);
}
// `count` (1 to 8) openings against prepared generator sets of one size and with one round count, as ONE job: every
// kernel of a round is launched once for all of them, so the late rounds have count times the waves.  u: opening i's
// challenges at u + i * rounds * 8.  zk_g1_open_end_batch delivers opening i's points at proof_host + i * (3 rounds + 1) * 36
// and its folded scalar at final_scalar_host + i * 8.
int zk_g1_open_begin_batch(void** handle, int count, const void* const* scalars, const void* const* prepared, const uint32_t* u, int rounds, void* stv) {
    ZK_ARG(count >= 1 && count <= OB_MAX, "zk_g1_open_begin_batch: 1 to 8 openings");
    ZK_ARG(scalars != nullptr && prepared != nullptr && u != nullptr, "zk_g1_open_begin_batch: null argument");
    OpenItem items[OB_MAX];
    size_t n = 0;
    for (int i = 0; i < count; ++i) {
        ZK_ARG(prepared[i] != nullptr && scalars[i] != nullptr, "zk_g1_open_begin_batch: null opening");
        const OpenPrepared* pr = (const OpenPrepared*)prepared[i];
        if (i == 0) n = pr->n;
        ZK_ARG(pr->n == n, "zk_g1_open_begin_batch: the generator sets differ in size");
        items[i] = OpenItem{scalars[i], nullptr, (const A29*)pr->a29, u + (size_t)i * rounds * 8, (const A29*)pr->comb, (const A29*)pr->comb2};
    }
    return open_begin_impl(handle, items, count, n, rounds, stv);
}
// zk_g1_open_begin_batch for vectors that are row folds of committed tensors: rows[i] holds tensor i's nrows[i] row
// commitments under the same generators, u_rows[i] the k_rows[i] challenges its rows were folded with (lowest row bit
// first, 2^k_rows >= nrows).  T of the first round is then the same combination of the row commitments -- equal as a group
// element to the sum over all generators that zk_g1_open_begin_batch computes, provided the commitments are the tensor's.
int zk_g1_open_begin_batch_rows(void** handle, int count, const void* const* scalars, const void* const* prepared, const uint32_t* u, int rounds,
                                const void* const* rows, const uint32_t* nrows, const uint32_t* const* u_rows, const int* k_rows, int cross_rounds, void* stv) {
    ZK_ARG(cross_rounds >= 0 && cross_rounds <= 4, "zk_g1_open_begin_batch_rows: 0 to 4 rounds of cross commitments");
    ZK_ARG(count >= 1 && count <= OB_MAX, "zk_g1_open_begin_batch_rows: 1 to 8 openings");
    ZK_ARG(scalars != nullptr && prepared != nullptr && u != nullptr && rows != nullptr && nrows != nullptr && u_rows != nullptr && k_rows != nullptr, "zk_g1_open_begin_batch_rows: null argument");
    OpenItem items[OB_MAX];
    size_t n = 0;
    for (int i = 0; i < count; ++i) {
        ZK_ARG(prepared[i] != nullptr && scalars[i] != nullptr && rows[i] != nullptr, "zk_g1_open_begin_batch_rows: null opening");
        ZK_ARG(nrows[i] >= 1 && k_rows[i] >= 0 && k_rows[i] <= 31 && ((uint64_t)1 << k_rows[i]) >= nrows[i] && (k_rows[i] == 0 || u_rows[i] != nullptr), "zk_g1_open_begin_batch_rows: rows and row challenges do not fit");
        const OpenPrepared* pr = (const OpenPrepared*)prepared[i];
        if (i == 0) n = pr->n;
        ZK_ARG(pr->n == n, "zk_g1_open_begin_batch_rows: the generator sets differ in size");
        items[i] = OpenItem{scalars[i], nullptr, (const A29*)pr->a29, u + (size_t)i * rounds * 8, (const A29*)pr->comb, (const A29*)pr->comb2, rows[i], nrows[i], u_rows[i], k_rows[i], cross_rounds,
                            (const A29*)pr->comb3};
    }
    return open_begin_impl(handle, items, count, n, rounds, stv);
}
int zk_g1_open_end_batch(void* handle, uint32_t* proof_host, uint32_t* final_scalar_host) { return zk_g1_open_end(handle, proof_host, final_scalar_host); }
int zk_g1_open_end(void* handle, uint32_t* proof_host, uint32_t* final_scalar_host) {
    ZK_ARG(handle != nullptr, "zk_g1_open_end: null handle");
    std::unique_ptr<OpenJob> job((OpenJob*)handle);
    launcher_wait(job->ticket);
    job->ticket = 0;
    int rc = job->queue_rc;
    if (rc) set_error(rc, job->queue_err);
    else rc = open_collect(*job, proof_host, final_scalar_host);
    if (rc) { (void)hipStreamSynchronize(job->st); (void)hipStreamSynchronize(job->aux); }
    job->arena.mark_idle();          // both streams have drained behind the job's last kernel
    (void)hipEventDestroy(job->ready);
    for (hipEvent_t e : job->events) (void)hipEventDestroy(e);
    return rc;
}

// Measurement: time every launch of the opening's fold kernel between begin and read with events on the launch stream.
static double g_fold_method_ms[3] = {0, 0, 0};
static unsigned long long g_fold_method_launches[3] = {0, 0, 0}, g_fold_method_pairs[3] = {0, 0, 0};
static double g_fold_method_mults[3] = {0, 0, 0};
int zk_prof_fold_begin(void) {
    for (auto& e : g_fold_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    g_fold_timer.ev.clear();
    g_fold_timer.method.clear();
    g_fold_timer.fp_mults = 0;
    g_fold_timer.pairs = 0;
    for (int m = 0; m < 3; ++m) { g_fold_timer.m_mults[m] = 0; g_fold_timer.m_pairs[m] = 0; }
    g_fold_timer.on = true;
    return 0;
}
// total_ms / launches: summed durations and number of timed launches; fp_mults: Fp multiplications they performed; pairs: pairs folded
int zk_prof_fold_read(double* total_ms, unsigned long long* launches, double* fp_mults, unsigned long long* pairs) {
    g_fold_timer.on = false;
    double tot = 0;
    for (int m = 0; m < 3; ++m) { g_fold_method_ms[m] = 0; g_fold_method_launches[m] = 0; }
    for (size_t i = 0; i < g_fold_timer.ev.size(); ++i) {
        auto& e = g_fold_timer.ev[i];
        ZK_HIP(hipEventSynchronize(e.second));
        float ms = 0;
        ZK_HIP(hipEventElapsedTime(&ms, e.first, e.second));
        tot += ms;
        const int m = i < g_fold_timer.method.size() ? g_fold_timer.method[i] : 0;
        g_fold_method_ms[m] += ms;
        g_fold_method_launches[m] += 1;
    }
    for (int m = 0; m < 3; ++m) { g_fold_method_mults[m] = g_fold_timer.m_mults[m]; g_fold_method_pairs[m] = g_fold_timer.m_pairs[m]; }
    *total_ms = tot;
    *launches = g_fold_timer.ev.size();
    *fp_mults = g_fold_timer.fp_mults;
    *pairs = g_fold_timer.pairs;
    for (auto& e : g_fold_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    g_fold_timer.ev.clear();
    g_fold_timer.method.clear();
    return 0;
}
// what the last zk_prof_fold_read counted, by method (0 walk, 1 comb, 2 three-round fold): ms, launches, pairs, Fp multiplications
int zk_prof_fold_methods(double* ms3, unsigned long long* launches3, unsigned long long* pairs3, double* fp_mults3) {
    for (int m = 0; m < 3; ++m) { ms3[m] = g_fold_method_ms[m]; launches3[m] = g_fold_method_launches[m]; pairs3[m] = g_fold_method_pairs[m]; fp_mults3[m] = g_fold_method_mults[m]; }
    return 0;
}

}  // extern "C"

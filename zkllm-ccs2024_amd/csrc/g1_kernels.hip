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
#include <cstring>
#include <vector>
#include "g1.hpp"
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

// ---- fixed-base table for commit_int -------------------------------------------------------------------------
// table (Jacobian, before normalisation): tab[(w * ngen + j) * half + (d-1)] = d * 2^(c*w) * G_j, d = 1..half
__global__ void __launch_bounds__(GT) k_msm_table(G1Jac* __restrict__ tab, const G1Jac* __restrict__ gens, size_t ngen, uint32_t c, uint32_t nwin) {
    const size_t j = (size_t)blockIdx.x * GT + threadIdx.x;
    if (j >= ngen) return;
    const uint32_t half = 1u << (c - 1);
    G1Jac base = gens[j];
    for (uint32_t w = 0; w < nwin; ++w) {
        G1Jac* row = tab + ((size_t)w * ngen + j) * half;
        G1Jac acc = base;
        row[0] = acc;
        for (uint32_t d = 1; d < half; ++d) { acc = g1_add(acc, base); row[d] = acc; }
        if (w + 1 < nwin) for (uint32_t k = 0; k < c; ++k) base = g1_double(base);
    }
}
// One workgroup per (row, segment): sum_j [s_j] G_j over the segment as mixed additions out of the
// affine table.  Scalars are embedded int32 values (commit_int_dev_func, commitment.cu:31-42).
__global__ void __launch_bounds__(GT) k_msm_rows(G1Jac* __restrict__ out, const G1Affine* __restrict__ tab, const int32_t* __restrict__ scalars,
                                                 size_t ngen, uint32_t c, uint32_t nwin, uint32_t nseg) {
    const size_t row = blockIdx.x;
    const uint32_t seg = blockIdx.y;
    const uint32_t half = 1u << (c - 1);
    const size_t per = (ngen + nseg - 1) / nseg;
    const size_t j0 = seg * per, j1 = (j0 + per < ngen) ? j0 + per : ngen;
    G1Jac acc = g1_infinity();
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
            G1Affine p = tab[((size_t)w * ngen + j) * half + (mag - 1)];
            if (nd) p.y = neg(p.y);
            acc = g1_add_mixed(acc, p);
        }
    }
    acc = block_sum_g1(acc);
    if (threadIdx.x == 0) out[row * nseg + seg] = acc;
}
__global__ void __launch_bounds__(256) k_fr_to_i32_checked(int32_t* __restrict__ out, uint32_t* __restrict__ bad, uint32_t* __restrict__ maxabs, const Fr* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const Fr x = in[i];
    // scalar_to_int semantics: values outside the int32 embedding collapse to what the reference reads
    const int32_t v = fr_to_i32(x);
    out[i] = v;
    const Fr back = fr_from_i64((int64_t)v);
    if (!equal(back, x)) atomicOr(bad, 1u);
    const uint32_t a = v < 0 ? (uint32_t)(-(int64_t)v) : (uint32_t)v;
    if (a) atomicMax(maxabs, a);
}

// ---- opening (me_open_step, commitment.cu:79-107) ------------------------------------------------------------------
// Five scalar multiplications per pair, one lane each: which = 0: [u](g0-g1), 1: [s0]g0, 2: [s1]g1, 3: [s0]g1, 4: [s1]g0.
// parts[which * new_size + pair].  Odd tail: 0: [u]g0, 1: [s0]g0, others infinity.
__global__ void __launch_bounds__(GT) k_open_parts(G1Jac* __restrict__ parts, const Fr* __restrict__ scalars, const G1Jac* __restrict__ gens, const Fr u, size_t old_size, size_t new_size) {
    const size_t t = (size_t)blockIdx.x * GT + threadIdx.x;
    if (t >= 5 * new_size) return;
    const uint32_t which = (uint32_t)(t / new_size);
    const size_t g = t % new_size;
    const size_t g0 = 2 * g, g1 = 2 * g + 1;
    G1Jac r = g1_infinity();
    if (g1 >= old_size) {
        if (which == 0) r = g1_mul(gens[g0], u);
        else if (which == 1) r = g1_mul(gens[g0], scalars[g0]);
    } else {
        switch (which) {
            case 0: r = g1_mul(g1_add(gens[g0], g1_neg(gens[g1])), u); break;
            case 1: r = g1_mul(gens[g0], scalars[g0]); break;
            case 2: r = g1_mul(gens[g1], scalars[g1]); break;
            case 3: r = g1_mul(gens[g1], scalars[g0]); break;
            default: r = g1_mul(gens[g0], scalars[g1]); break;
        }
    }
    parts[t] = r;
}
// new_gens = g1 + part0 (or part0 on the odd tail); T = part1 + part2 (in place in part1); new scalars
__global__ void __launch_bounds__(GT) k_open_combine(Fr* __restrict__ new_scalars, G1Jac* __restrict__ new_gens, G1Jac* __restrict__ parts,
                                                     const Fr* __restrict__ scalars, const G1Jac* __restrict__ gens, const Fr u_mont, size_t old_size, size_t new_size) {
    const size_t g = (size_t)blockIdx.x * GT + threadIdx.x;
    if (g >= new_size) return;
    const size_t g0 = 2 * g, g1 = 2 * g + 1;
    if (g1 >= old_size) {
        new_scalars[g] = sub(scalars[g0], mont_mul(u_mont, scalars[g0]));
        new_gens[g] = parts[g];
        return;
    }
    new_scalars[g] = add(scalars[g0], mont_mul(u_mont, sub(scalars[g1], scalars[g0])));
    new_gens[g] = g1_add(gens[g1], parts[g]);
    parts[new_size + g] = g1_add(parts[new_size + g], parts[2 * new_size + g]);
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
    Scratch part(sizeof(G1Jac) * nseg);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_g1_rowsum, dim3(1, nseg), dim3(GT), 0, st, part.as<G1Jac>(), in, n, nseg);
    hipLaunchKernelGGL(k_g1_rowsum, dim3(1, 1), dim3(GT), 0, st, out, part.as<G1Jac>(), (size_t)nseg, 1u);
    ZK_LAUNCH_CHECK();
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
    Scratch res(sizeof(G1Jac));
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
    Scratch part(sizeof(G1Jac) * nrow * nseg);
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
        if (!bufs[which]) rc = pool_alloc(&bufs[which], sizeof(G1Jac) * out_n);
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
    for (int i = 0; i < 2; ++i) if (bufs[i]) pool_free(bufs[i]);
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
    Scratch ints(sizeof(int32_t) * total), flags(8);
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
    Scratch tabj(sizeof(G1Jac) * tab_n), taba(sizeof(G1Affine) * tab_n);
    if (tabj.rc) return tabj.rc;
    if (taba.rc) return taba.rc;
    hipLaunchKernelGGL(k_msm_table, dim3(cdiv(ngen, GT)), dim3(GT), 0, st, tabj.as<G1Jac>(), (const G1Jac*)gens, ngen, c, nwin);
    hipLaunchKernelGGL(k_g1_normalize<true>, dim3(cdiv(cdiv(tab_n, CH), GT)), dim3(GT), 0, st, taba.p, tabj.as<G1Jac>(), tab_n);
    ZK_LAUNCH_CHECK();
    uint32_t nseg = 1;
    if (m < 2048) { nseg = (uint32_t)(2048 / m); const uint32_t cap = (uint32_t)((ngen + GT - 1) / GT); if (nseg > cap) nseg = cap; if (nseg < 1) nseg = 1; }
    if (nseg == 1) {
        hipLaunchKernelGGL(k_msm_rows, dim3((unsigned)m, 1), dim3(GT), 0, st, (G1Jac*)out, taba.as<G1Affine>(), ints.as<int32_t>(), ngen, c, nwin, 1u);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    Scratch part(sizeof(G1Jac) * m * nseg);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_msm_rows, dim3((unsigned)m, nseg), dim3(GT), 0, st, part.as<G1Jac>(), taba.as<G1Affine>(), ints.as<int32_t>(), ngen, c, nwin, nseg);
    hipLaunchKernelGGL(k_g1_rowsum, dim3((unsigned)m, 1), dim3(GT), 0, st, (G1Jac*)out, part.as<G1Jac>(), (size_t)nseg, 1u);
    ZK_LAUNCH_CHECK();
    return 0;
}

// One round of Commitment::me_open (commitment.cu:79-129).  u: standard-form challenge (used both as the
// field scalar of the fold and as the raw 256-bit integer of the scalar multiplications, as the reference does).
// new_scalars / new_gens: (old_size+1)/2 elements.  sums_host: 3 points (sum T, sum T0, sum T1).
int zk_g1_open_round(void* new_scalars, void* new_gens, uint32_t* sums_host, const void* scalars, const void* gens, const uint32_t* u, size_t old_size, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(old_size >= 1, "zk_g1_open_round: empty input");
    const size_t new_size = (old_size + 1) / 2;
    Scratch parts(sizeof(G1Jac) * 5 * new_size), sums(sizeof(G1Jac) * 3);
    if (parts.rc) return parts.rc;
    if (sums.rc) return sums.rc;
    const Fr uu = load_fr(u);
    hipLaunchKernelGGL(k_open_parts, dim3(cdiv(5 * new_size, GT)), dim3(GT), 0, st, parts.as<G1Jac>(), (const Fr*)scalars, (const G1Jac*)gens, uu, old_size, new_size);
    hipLaunchKernelGGL(k_open_combine, dim3(cdiv(new_size, GT)), dim3(GT), 0, st, (Fr*)new_scalars, (G1Jac*)new_gens, parts.as<G1Jac>(), (const Fr*)scalars, (const G1Jac*)gens, to_mont(uu), old_size, new_size);
    ZK_LAUNCH_CHECK();
    G1Jac* P = parts.as<G1Jac>();
    int rc = g1_sum_device(sums.as<G1Jac>() + 0, P + 1 * new_size, new_size, st);
    if (!rc) rc = g1_sum_device(sums.as<G1Jac>() + 1, P + 3 * new_size, new_size, st);
    if (!rc) rc = g1_sum_device(sums.as<G1Jac>() + 2, P + 4 * new_size, new_size, st);
    if (rc) return rc;
    void* stage = nullptr;
    rc = staging(&stage, sizeof(G1Jac) * 3);
    if (rc) return rc;
    ZK_HIP(hipMemcpyAsync(stage, sums.p, sizeof(G1Jac) * 3, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    memcpy(sums_host, stage, sizeof(G1Jac) * 3);
    return 0;
}

}  // extern "C"

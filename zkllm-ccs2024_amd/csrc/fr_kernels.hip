// FrTensor kernels for gfx950: elementwise, conversions, layout, sums, multilinear folds and
// the inner-product sumcheck rounds.  Tensors hold standard-form residues, 32 B per element
// (8 little-endian u32 limbs), exactly the reference's Fr_t layout (fr-tensor.cu:181-184).
//
// Differences from the reference's kernels that do not change any output byte:
//  * broadcast operands and challenges are converted to Montgomery form once on the host, so a
//    product with them costs one Montgomery multiplication instead of two;
//  * sums of products are accumulated with the R^-1 factor still attached and corrected once;
//  * folds run several levels per pass (registers) and finish in one workgroup (LDS).
#include <cstring>
#include <mutex>
#include "field.hpp"
#include "rt.hpp"
#include "../../include/zkllm_hip.h"

using namespace zk;

static constexpr int TPB = 256;

// ------------------------------------------------------------------------------------------------
// elementwise (fr-tensor.cu:71-153)
// ------------------------------------------------------------------------------------------------
enum { EW_ADD = 0, EW_SUB = 1, EW_MUL = 2, EW_MONTMUL = 3 };

template <int OP> __global__ void __launch_bounds__(TPB) k_ew(Fr* __restrict__ out, const Fr* __restrict__ a, const Fr* __restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const Fr x = a[i], y = b[i];
    Fr r;
    if (OP == EW_ADD) r = add(x, y);
    else if (OP == EW_SUB) r = sub(x, y);
    else if (OP == EW_MUL) r = fr_mul_std(x, y);
    else r = mont_mul(x, y);
    out[i] = r;
}
// s: for EW_MUL the scalar is already in Montgomery form (s*R), so one mont_mul yields a*s.
template <int OP> __global__ void __launch_bounds__(TPB) k_ew_s(Fr* __restrict__ out, const Fr* __restrict__ a, const Fr s, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const Fr x = a[i];
    Fr r;
    if (OP == EW_ADD) r = add(x, s);
    else if (OP == EW_SUB) r = sub(x, s);
    else r = mont_mul(x, s);
    out[i] = r;
}
__global__ void __launch_bounds__(TPB) k_neg(Fr* __restrict__ out, const Fr* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = neg(a[i]);
}
__global__ void __launch_bounds__(TPB) k_fill(Fr* __restrict__ out, const Fr s, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = s;
}
// Z[i] += bias[i % cols] (zkfc.cu:36-41)
__global__ void __launch_bounds__(TPB) k_bias(Fr* __restrict__ z, const Fr* __restrict__ bias, size_t n, uint32_t cols) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) z[i] = add(z[i], bias[i % cols]);
}

// ------------------------------------------------------------------------------------------------
// conversions (fr-tensor.cu:186-208, 691-775, 922-945)
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(TPB) k_from_i32(Fr* __restrict__ out, const int32_t* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_from_i64((int64_t)in[i]);
}
__global__ void __launch_bounds__(TPB) k_from_i64(Fr* __restrict__ out, const int64_t* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_from_i64(in[i]);
}
__global__ void __launch_bounds__(TPB) k_from_u32(Fr* __restrict__ out, const uint32_t* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_from_u64((uint64_t)in[i]);
}
// round half away from zero after scaling (float_to_scalar / double_to_scalar)
__global__ void __launch_bounds__(TPB) k_from_f32(Fr* __restrict__ out, const float* __restrict__ in, uint64_t sf, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    float x = in[i] * (float)sf;
    const int64_t v = (x >= 0) ? (int64_t)((double)x + 0.5) : (int64_t)((double)x - 0.5);
    out[i] = fr_from_i64(v);
}
__global__ void __launch_bounds__(TPB) k_from_f64(Fr* __restrict__ out, const double* __restrict__ in, uint64_t sf, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    double x = in[i] * (double)sf;
    const int64_t v = (x >= 0) ? (int64_t)(x + 0.5) : (int64_t)(x - 0.5);
    out[i] = fr_from_i64(v);
}
__global__ void __launch_bounds__(TPB) k_to_i32(int32_t* __restrict__ out, const Fr* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_to_i32(in[i]);
}
__global__ void __launch_bounds__(TPB) k_to_i64(int64_t* __restrict__ out, const Fr* __restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = fr_to_i64(in[i]);
}

// ------------------------------------------------------------------------------------------------
// layout (fr-tensor.cu:800-828 pad, :885-900 transpose; tlookup.cu:446-453 gather)
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(TPB) k_pad(Fr* __restrict__ out, const Fr* __restrict__ in, size_t n_out, uint32_t last_in, uint32_t last_out, const Fr pad) {
    const size_t g = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (g >= n_out) return;
    const size_t g0 = g / last_out;
    const uint32_t g1 = (uint32_t)(g % last_out);
    out[g] = (g1 >= last_in) ? pad : in[g0 * last_in + g1];
}
// 32x32 tile through LDS so both the read and the write are contiguous along the fast axis
// blockIdx.z selects one of a stack of M x N matrices
__global__ void __launch_bounds__(TPB) k_transpose(Fr* __restrict__ out, const Fr* __restrict__ in, uint32_t M, uint32_t N) {
    __shared__ uint32_t tile[8][32][33];
    in += (size_t)blockIdx.z * M * N;
    out += (size_t)blockIdx.z * M * N;
    const uint32_t bx = blockIdx.x * 32, by = blockIdx.y * 32;
    const uint32_t tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    for (uint32_t r = ty; r < 32; r += 8) {
        const uint32_t row = by + r, col = bx + tx;
        if (row < M && col < N) {
            const Fr v = in[(size_t)row * N + col];
#pragma unroll
            for (int l = 0; l < 8; ++l) tile[l][r][tx] = v.v[l];
        }
    }
    __syncthreads();
    for (uint32_t r = ty; r < 32; r += 8) {
        const uint32_t col = bx + r, row = by + tx;     // output row = input col
        if (row < M && col < N) {
            Fr v;
#pragma unroll
            for (int l = 0; l < 8; ++l) v.v[l] = tile[l][tx][r];
            out[(size_t)col * M + row] = v;
        }
    }
}
__global__ void __launch_bounds__(TPB) k_gather(Fr* __restrict__ out, const Fr* __restrict__ table, const uint32_t* __restrict__ idx, size_t n) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) out[i] = table[idx[i]];
}

// ------------------------------------------------------------------------------------------------
// block reduction of K running sums per thread; partials[k * gridDim.x + blockIdx.x]
// ------------------------------------------------------------------------------------------------
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
// one block per k: out[k] = sum of partials[k*nb .. k*nb+nb)
__global__ void __launch_bounds__(TPB) k_finish_sums(Fr* __restrict__ out, const Fr* __restrict__ partials, uint32_t nb) {
    Fr acc[1] = {big_zero<8>()};
    const Fr* p = partials + (size_t)blockIdx.x * nb;
    for (uint32_t i = threadIdx.x; i < nb; i += TPB) acc[0] = add(acc[0], p[i]);
    block_reduce_store<1>(acc, out);   // gridDim.x == K, so out[0*K + blockIdx.x] = out[k]
}

__global__ void __launch_bounds__(TPB) k_sum(Fr* __restrict__ partials, const Fr* __restrict__ a, size_t n) {
    Fr acc[1] = {big_zero<8>()};
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (size_t)gridDim.x * TPB) acc[0] = add(acc[0], a[i]);
    block_reduce_store<1>(acc, partials);
}
// sum_i a_i*b_i*R^-1 (the caller applies the R^2 correction once)
__global__ void __launch_bounds__(TPB) k_dot(Fr* __restrict__ partials, const Fr* __restrict__ a, const Fr* __restrict__ b, size_t n) {
    Fr acc[1] = {big_zero<8>()};
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (size_t)gridDim.x * TPB) acc[0] = add(acc[0], mont_mul(a[i], b[i]));
    block_reduce_store<1>(acc, partials);
}

static inline unsigned reduce_grid(size_t n) {
    size_t b = (n + TPB - 1) / TPB;
    if (b > 2048) b = 2048;
    if (b < 1) b = 1;
    return (unsigned)b;
}
// finish K sums living in `partials` (K x nb) and bring them to the host (standard layout)
template <int K> static int finish_to_host(Fr* partials, unsigned nb, Fr* host_out, hipStream_t st) {
    void* stage = nullptr;
    int rc = staging(&stage, sizeof(Fr) * K);
    if (rc) return rc;
    Scratch fin(sizeof(Fr) * K, st);
    if (fin.rc) return fin.rc;
    hipLaunchKernelGGL(k_finish_sums, dim3(K), dim3(TPB), 0, st, fin.as<Fr>(), partials, nb);
    ZK_LAUNCH_CHECK();
    ZK_HIP(hipMemcpyAsync(stage, fin.p, sizeof(Fr) * K, hipMemcpyDeviceToHost, st));
    ZK_HIP(hipStreamSynchronize(st));
    memcpy(host_out, stage, sizeof(Fr) * K);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// multilinear folds
// ------------------------------------------------------------------------------------------------
template <int L> struct FrPack { Fr x[L]; };

// Folds L levels of the middle axis of in[other][cur][window] (adjacent pairs along `cur`, index
// bit 0 first; positions past `cur` read as zero, which is the reference's odd-tail rule
// a - x*a).  xs are in Montgomery form.  (fr-tensor.cu:518-560, 588-626)
template <int L> __global__ void __launch_bounds__(TPB)
k_fold_axis(Fr* __restrict__ out, const Fr* __restrict__ in, const FrPack<L> xs, size_t n_out, uint32_t cur, uint32_t cur_out, size_t window) {
    const size_t g = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (g >= n_out) return;
    const size_t i2 = g % window;
    const size_t t = g / window;
    const uint32_t i1 = (uint32_t)(t % cur_out);
    const size_t i0 = t / cur_out;
    const Fr* base = in + (i0 * cur) * window + i2;
    const uint32_t first = i1 << L;
    Fr v[1 << L];
#pragma unroll
    for (int j = 0; j < (1 << L); ++j) v[j] = (first + j < cur) ? base[(size_t)(first + j) * window] : big_zero<8>();
#pragma unroll
    for (int l = 0; l < L; ++l) {
#pragma unroll
        for (int j = 0; j < (1 << (L - 1 - l)); ++j) v[j] = add(v[2 * j], mont_mul(xs.x[l], sub(v[2 * j + 1], v[2 * j])));
    }
    out[g] = v[0];
}
// The same L levels as one weighted sum: out = sum_j w_j in_j with w_j = prod_l (x_l if bit l of j else 1 - x_l), the
// products of every four terms sharing one Montgomery reduction (8 x 64 + 2 x 72 multiply-adds for three levels instead of
// 7 x 136).  The field value, hence the canonical result, is that of the level-by-level fold.  ws in Montgomery form.
template <int L> __global__ void __launch_bounds__(TPB)
k_fold_axis_dot(Fr* __restrict__ out, const Fr* __restrict__ in, const FrPack<(1 << L)> ws, size_t n_out, uint32_t cur, uint32_t cur_out, size_t window) {
    static_assert(L >= 2, "groups of four terms");
    const size_t g = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (g >= n_out) return;
    const size_t i2 = g % window;
    const size_t t = g / window;
    const uint32_t i1 = (uint32_t)(t % cur_out);
    const size_t i0 = t / cur_out;
    const Fr* base = in + (i0 * cur) * window + i2;
    const uint32_t first = i1 << L;
    Fr acc;
#pragma unroll
    for (int q = 0; q < (1 << L); q += 4) {
        Fr v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = (first + q + j < cur) ? base[(size_t)(first + q + j) * window] : big_zero<8>();
        const Fr part = mont_dot<8, 4>(v, ws.x + q);
        acc = q ? add(acc, part) : part;
    }
    out[g] = acc;
}

// Finishes a multilinear evaluation inside one workgroup: n <= 1024 values, k levels.
struct FrPack12 { Fr x[12]; };
static constexpr uint32_t ME_SMALL_MAX = 1024;
__global__ void __launch_bounds__(TPB) k_me_small(Fr* __restrict__ out, const Fr* __restrict__ in, const FrPack12 xs, uint32_t n, uint32_t k) {
    __shared__ uint32_t buf[8][ME_SMALL_MAX];
    const uint32_t t = threadIdx.x;
    for (uint32_t i = t; i < ME_SMALL_MAX; i += TPB) {
        Fr v = (i < n) ? in[i] : big_zero<8>();
#pragma unroll
        for (int l = 0; l < 8; ++l) buf[l][i] = v.v[l];
    }
    __syncthreads();
    uint32_t cur = 1u << k;    // zero-extended length
    for (uint32_t lvl = 0; lvl < k; ++lvl) {
        const uint32_t half = cur >> 1;
        Fr r[ME_SMALL_MAX / 2 / TPB];
        int cnt = 0;
        for (uint32_t j = t; j < half; j += TPB, ++cnt) {
            Fr a, b;
#pragma unroll
            for (int l = 0; l < 8; ++l) { a.v[l] = buf[l][2 * j]; b.v[l] = buf[l][2 * j + 1]; }
            r[cnt] = add(a, mont_mul(xs.x[lvl], sub(b, a)));
        }
        __syncthreads();
        cnt = 0;
        for (uint32_t j = t; j < half; j += TPB, ++cnt) {
#pragma unroll
            for (int l = 0; l < 8; ++l) buf[l][j] = r[cnt].v[l];
        }
        __syncthreads();
        cur = half;
    }
    if (t == 0) {
        Fr v;
#pragma unroll
        for (int l = 0; l < 8; ++l) v.v[l] = buf[l][0];
        out[0] = v;
    }
}

// MSB fold of the zero-extended vector: out[i] = a[i] + v*(a[i+n_out] - a[i])  (zkfc.cu:113-127,
// tlookup.cu:94-103, proof.cu:180-188)
__global__ void __launch_bounds__(TPB) k_fold_halves(Fr* __restrict__ out, const Fr* __restrict__ a, const Fr v_mont, size_t n_in, size_t n_out) {
    const size_t g = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (g >= n_out) return;
    const Fr a0 = (g < n_in) ? a[g] : big_zero<8>();
    const Fr a1 = (g + n_out < n_in) ? a[g + n_out] : big_zero<8>();
    out[g] = add(a0, mont_mul(v_mont, sub(a1, a0)));
}
// Stacked variant over [N][D] (zkfc.cu:169-185): same formula on whole rows
// (covered by k_fold_halves with n_in = N*D, n_out = N_out*D).

// ------------------------------------------------------------------------------------------------
// inner-product sumcheck (zkfc.cu:94-151)
// ------------------------------------------------------------------------------------------------
// Three sums of one round, each still carrying R^-1:
//   s0 = sum a0*b0, s1 = sum a0*(b1-b0) + b0*(a1-a0), s2 = sum (a1-a0)*(b1-b0)
__global__ void __launch_bounds__(TPB) k_ip_round(Fr* __restrict__ partials, const Fr* __restrict__ a, const Fr* __restrict__ b, size_t n_in, size_t n_out) {
    Fr acc[3] = {big_zero<8>(), big_zero<8>(), big_zero<8>()};
    for (size_t g = (size_t)blockIdx.x * TPB + threadIdx.x; g < n_out; g += (size_t)gridDim.x * TPB) {
        const Fr a0 = (g < n_in) ? a[g] : big_zero<8>();
        const Fr b0 = (g < n_in) ? b[g] : big_zero<8>();
        const Fr a1 = (g + n_out < n_in) ? a[g + n_out] : big_zero<8>();
        const Fr b1 = (g + n_out < n_in) ? b[g + n_out] : big_zero<8>();
        const Fr da = sub(a1, a0), db = sub(b1, b0);
        acc[0] = add(acc[0], mont_mul(a0, b0));
        acc[1] = add(acc[1], add(mont_mul(a0, db), mont_mul(b0, da)));
        acc[2] = add(acc[2], mont_mul(da, db));
    }
    block_reduce_store<3>(acc, partials);
}

// Stacked form (zkip_stacked_poly_kernel zkfc.cu:153-167 followed by the multilinear evaluation over the
// stacking axis, zkfc.cu:187-209): tensors are [N][D], halves are taken over N, and row n of the three
// term tensors is weighted by E[n] (eq table, Montgomery form) before everything is summed.
__global__ void __launch_bounds__(TPB) k_ip_round_w(Fr* __restrict__ partials, const Fr* __restrict__ a, const Fr* __restrict__ b, const Fr* __restrict__ E,
                                                    size_t D, size_t n_in, size_t n_out) {
    Fr acc[3] = {big_zero<8>(), big_zero<8>(), big_zero<8>()};
    for (size_t g = (size_t)blockIdx.x * TPB + threadIdx.x; g < n_out; g += (size_t)gridDim.x * TPB) {
        const Fr a0 = (g < n_in) ? a[g] : big_zero<8>();
        const Fr b0 = (g < n_in) ? b[g] : big_zero<8>();
        const Fr a1 = (g + n_out < n_in) ? a[g + n_out] : big_zero<8>();
        const Fr b1 = (g + n_out < n_in) ? b[g + n_out] : big_zero<8>();
        const Fr da = sub(a1, a0), db = sub(b1, b0);
        const Fr e = E[g / D];
        acc[0] = add(acc[0], mont_mul(e, mont_mul(a0, b0)));
        acc[1] = add(acc[1], mont_mul(e, add(mont_mul(a0, db), mont_mul(b0, da))));
        acc[2] = add(acc[2], mont_mul(e, mont_mul(da, db)));
    }
    block_reduce_store<3>(acc, partials);
}

// Whole sumcheck in one workgroup for short vectors (n <= 8192): every round's three sums are
// written to polys[round*3 + {0,1,2}] (standard form, R^2-corrected), the folded vectors
// ping-pong through `work` (2 * 2 * n_pow2/2 elements) and the final a, b land in fin[0..1].
// Challenges are consumed from the back of vs (Montgomery form), as the reference does.
struct FrPack16 { Fr x[16]; };
__global__ void __launch_bounds__(1024) k_ip_small(Fr* __restrict__ polys, Fr* __restrict__ fin, Fr* __restrict__ work,
                                                   const Fr* __restrict__ a_in, const Fr* __restrict__ b_in, const FrPack16 vs, uint32_t n, uint32_t k) {
    __shared__ uint32_t red[8][1024];
    const uint32_t t = threadIdx.x;
    const uint32_t half0 = (1u << k) >> 1;
    const Fr* a = a_in;
    const Fr* b = b_in;
    uint32_t n_in = n;
    const Fr r2 = big_r2<8>();
    for (uint32_t round = 0; round < k; ++round) {
        const uint32_t n_out = (1u << (k - round)) >> 1;
        Fr* na = work + (size_t)(round & 1) * 2 * half0;
        Fr* nb = na + half0;
        const Fr v = vs.x[k - 1 - round];
        Fr acc[3] = {big_zero<8>(), big_zero<8>(), big_zero<8>()};
        for (uint32_t g = t; g < n_out; g += 1024) {
            const Fr a0 = (g < n_in) ? a[g] : big_zero<8>();
            const Fr b0 = (g < n_in) ? b[g] : big_zero<8>();
            const Fr a1 = (g + n_out < n_in) ? a[g + n_out] : big_zero<8>();
            const Fr b1 = (g + n_out < n_in) ? b[g + n_out] : big_zero<8>();
            const Fr da = sub(a1, a0), db = sub(b1, b0);
            acc[0] = add(acc[0], mont_mul(a0, b0));
            acc[1] = add(acc[1], add(mont_mul(a0, db), mont_mul(b0, da)));
            acc[2] = add(acc[2], mont_mul(da, db));
            na[g] = add(a0, mont_mul(v, da));
            nb[g] = add(b0, mont_mul(v, db));
        }
        for (int q = 0; q < 3; ++q) {
#pragma unroll
            for (int l = 0; l < 8; ++l) red[l][t] = acc[q].v[l];
            __syncthreads();
            for (uint32_t s = 512; s > 0; s >>= 1) {
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
                polys[round * 3 + q] = mont_mul(x, r2);
            }
            __syncthreads();
        }
        a = na; b = nb; n_in = n_out;
    }
    if (t == 0) { fin[0] = a[0]; fin[1] = b[0]; }
}

// ------------------------------------------------------------------------------------------------
// host side of the C ABI
// ------------------------------------------------------------------------------------------------
static inline Fr load_fr(const uint32_t* p) { Fr r; memcpy(&r, p, 32); return r; }

#define LAUNCH1D(kernel, n, st, ...)                                                         \
    do {                                                                                     \
        if ((n) > 0) {                                                                       \
            hipLaunchKernelGGL(kernel, dim3(cdiv((n), TPB)), dim3(TPB), 0, (hipStream_t)(st), __VA_ARGS__); \
            ZK_LAUNCH_CHECK();                                                               \
        }                                                                                    \
    } while (0)

// out[r] = sum_j (x_rj / scale)^2 in double precision, the terms added one after the other from j = 0 (the order a plain
// host loop uses, so the rounding is the same).  One wave per row: the lanes form 64 terms at a time -- conversion,
// division and square are exactly rounded operations -- and lane 0 adds them in order.
__global__ void __launch_bounds__(64) k_row_sumsq_f64(double* __restrict__ out, const Fr* __restrict__ X, uint32_t cols, double scale) {
    __shared__ double term[64];
    const uint32_t r = blockIdx.x, t = threadIdx.x;
    const Fr* row = X + (size_t)r * cols;
    double acc = 0.0;
    for (uint32_t j0 = 0; j0 < cols; j0 += 64) {
        const uint32_t j = j0 + t;
        double v = 0.0;
        if (j < cols) {
            const double x = (double)fr_to_i64(row[j]) / scale;
            v = x * x;
        }
        term[t] = v;
        __syncthreads();
        if (t == 0) {
            const uint32_t cnt = cols - j0 < 64u ? cols - j0 : 64u;
            for (uint32_t q = 0; q < cnt; ++q) acc += term[q];
        }
        __syncthreads();
    }
    if (t == 0) out[r] = acc;
}

// ------------------------------------------------------------------------------------------------
// FrTensor::sum for callers that cannot allocate (code under stream capture, serving loops, harnesses that forbid
// hipMalloc).  The block partials of k_sum live in a file-scope device array instead of a pool block; the result goes
// to a device element of the caller's.  The array is one per GPU and is shared by every call on that GPU: calls that
// overlap on one GPU (two streams, two threads) race on it.  k_sum writes every partial that k_finish_sums reads, so
// nothing has to be cleared between calls.
// ------------------------------------------------------------------------------------------------
static constexpr unsigned SUM_STATIC_MAX_BLOCKS = 2048;                 // reduce_grid's cap
static constexpr int SUM_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) uint32_t scratch[SUM_STATIC_MAX_BLOCKS * 8];   // 64 KiB of block partials

static std::mutex g_scratch_mu;
static Fr* g_scratch_ptr[SUM_STATIC_MAX_DEVICES] = {};

// Address of this device's copy of `scratch` (the array's name is only a host-side handle), resolved once per device.
static int scratch_address(Fr** out) {
    int dev = -1;
    ZK_HIP(hipGetDevice(&dev));
    ZK_ARG(dev >= 0 && dev < SUM_STATIC_MAX_DEVICES, "zk_fr_sum_static: device index over 63");
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        ZK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        ZK_ARG(p != nullptr, "zk_fr_sum_static: the scratch array has no device address");
        g_scratch_ptr[dev] = (Fr*)p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
namespace zk {
int fr_static_scratch_setup() { Fr* p = nullptr; return scratch_address(&p); }
}

extern "C" {

int zk_fr_add(void* out, const void* a, const void* b, size_t n, void* st) { LAUNCH1D(k_ew<EW_ADD>, n, st, (Fr*)out, (const Fr*)a, (const Fr*)b, n); return 0; }
int zk_fr_sub(void* out, const void* a, const void* b, size_t n, void* st) { LAUNCH1D(k_ew<EW_SUB>, n, st, (Fr*)out, (const Fr*)a, (const Fr*)b, n); return 0; }
int zk_fr_mul(void* out, const void* a, const void* b, size_t n, void* st) { LAUNCH1D(k_ew<EW_MUL>, n, st, (Fr*)out, (const Fr*)a, (const Fr*)b, n); return 0; }
int zk_fr_montmul(void* out, const void* a, const void* b, size_t n, void* st) { LAUNCH1D(k_ew<EW_MONTMUL>, n, st, (Fr*)out, (const Fr*)a, (const Fr*)b, n); return 0; }
int zk_fr_neg(void* out, const void* a, size_t n, void* st) { LAUNCH1D(k_neg, n, st, (Fr*)out, (const Fr*)a, n); return 0; }
int zk_fr_add_s(void* out, const void* a, const uint32_t* s, size_t n, void* st) { LAUNCH1D(k_ew_s<EW_ADD>, n, st, (Fr*)out, (const Fr*)a, load_fr(s), n); return 0; }
int zk_fr_sub_s(void* out, const void* a, const uint32_t* s, size_t n, void* st) { LAUNCH1D(k_ew_s<EW_SUB>, n, st, (Fr*)out, (const Fr*)a, load_fr(s), n); return 0; }
int zk_fr_mul_s(void* out, const void* a, const uint32_t* s, size_t n, void* st) {
    const Fr sm = to_mont(load_fr(s));
    LAUNCH1D(k_ew_s<EW_MUL>, n, st, (Fr*)out, (const Fr*)a, sm, n);
    return 0;
}
// a*R (Scalar_mont) is a Montgomery product with R^2; a*R^-1 (Scalar_unmont) one with 1.
int zk_fr_mont(void* out, const void* a, size_t n, void* st) { LAUNCH1D(k_ew_s<EW_MUL>, n, st, (Fr*)out, (const Fr*)a, big_r2<8>(), n); return 0; }
int zk_fr_unmont(void* out, const void* a, size_t n, void* st) {
    Fr one = big_zero<8>(); one.v[0] = 1;
    LAUNCH1D(k_ew_s<EW_MUL>, n, st, (Fr*)out, (const Fr*)a, one, n);
    return 0;
}
int zk_fr_fill(void* out, const uint32_t* s, size_t n, void* st) { LAUNCH1D(k_fill, n, st, (Fr*)out, load_fr(s), n); return 0; }
int zk_fr_bias_add(void* z, const void* bias, size_t rows, uint32_t cols, void* st) {
    ZK_ARG(cols > 0, "zk_fr_bias_add: cols == 0");
    LAUNCH1D(k_bias, rows * cols, st, (Fr*)z, (const Fr*)bias, rows * cols, cols);
    return 0;
}

int zk_fr_from_i32(void* out, const void* in, size_t n, void* st) { LAUNCH1D(k_from_i32, n, st, (Fr*)out, (const int32_t*)in, n); return 0; }
int zk_fr_from_i64(void* out, const void* in, size_t n, void* st) { LAUNCH1D(k_from_i64, n, st, (Fr*)out, (const int64_t*)in, n); return 0; }
int zk_fr_from_u32(void* out, const void* in, size_t n, void* st) { LAUNCH1D(k_from_u32, n, st, (Fr*)out, (const uint32_t*)in, n); return 0; }
int zk_fr_from_f32(void* out, const void* in, uint64_t sf, size_t n, void* st) { LAUNCH1D(k_from_f32, n, st, (Fr*)out, (const float*)in, sf, n); return 0; }
int zk_fr_from_f64(void* out, const void* in, uint64_t sf, size_t n, void* st) { LAUNCH1D(k_from_f64, n, st, (Fr*)out, (const double*)in, sf, n); return 0; }
int zk_fr_to_i32(void* out, const void* in, size_t n, void* st) { LAUNCH1D(k_to_i32, n, st, (int32_t*)out, (const Fr*)in, n); return 0; }
// sums of squares of the rows of a rows x cols tensor of small signed integers, each divided by `scale` first, in double
// precision with the terms added in index order (the mean square of RMSNorm as a host loop would compute it;
// llama-rmsnorm.py:38-39 computes it with torch before the prover runs).  out_f64: rows doubles on the device.
int zk_row_sumsq_f64(void* out_f64, const void* X, uint32_t rows, uint32_t cols, double scale, void* st) {
    if (rows == 0) return 0;
    ZK_ARG(cols >= 1 && scale != 0.0, "zk_row_sumsq_f64: empty rows or zero scale");
    hipLaunchKernelGGL(k_row_sumsq_f64, dim3(rows), dim3(64), 0, (hipStream_t)st, (double*)out_f64, (const Fr*)X, cols, scale);
    ZK_LAUNCH_CHECK();
    return 0;
}
int zk_fr_to_i64(void* out, const void* in, size_t n, void* st) { LAUNCH1D(k_to_i64, n, st, (int64_t*)out, (const Fr*)in, n); return 0; }

int zk_fr_pad(void* out, const void* in, size_t rows, uint32_t last_in, uint32_t last_out, const uint32_t* pad, void* st) {
    ZK_ARG(last_in > 0 && last_out >= last_in, "zk_fr_pad: need 0 < last_in <= last_out");
    const size_t n_out = rows * last_out;
    LAUNCH1D(k_pad, n_out, st, (Fr*)out, (const Fr*)in, n_out, last_in, last_out, load_fr(pad));
    return 0;
}
int zk_fr_transpose_batched(void* out, const void* in, uint32_t batch, uint32_t M, uint32_t N, void* st) {
    if (batch == 0 || M == 0 || N == 0) return 0;
    ZK_ARG(out != in, "zk_fr_transpose: in-place transpose is not supported");
    ZK_ARG(batch <= 65535 && cdiv(M, 32) <= 65535, "zk_fr_transpose: too many matrices or rows for one launch");
    hipLaunchKernelGGL(k_transpose, dim3(cdiv(N, 32), cdiv(M, 32), batch), dim3(TPB), 0, (hipStream_t)st, (Fr*)out, (const Fr*)in, M, N);
    ZK_LAUNCH_CHECK();
    return 0;
}
int zk_fr_transpose(void* out, const void* in, uint32_t M, uint32_t N, void* st) { return zk_fr_transpose_batched(out, in, 1, M, N, st); }
// out[b][a][c] = in[a][b][c]: the leading two axes of a three-axis tensor swapped, rows of C elements moved whole (what two
// transposes do to bring [token][head][k] to [head][token][k] and back, in one pass)
// a workgroup per output row (b, a): the row's position is worked out once, by the scalar unit, and the lanes move its 16-byte words
__global__ void __launch_bounds__(TPB) k_swap_axes(uint4* __restrict__ out, const uint4* __restrict__ in, uint32_t A, uint32_t B, uint32_t Cw) {
    const uint32_t ba = blockIdx.x, a = ba % A, b = ba / A;
    const uint4* __restrict__ src = in + ((size_t)a * B + b) * Cw;
    uint4* __restrict__ dst = out + (size_t)ba * Cw;
    for (uint32_t w = threadIdx.x; w < Cw; w += TPB) dst[w] = src[w];
}
int zk_fr_swap_axes(void* out, const void* in, uint32_t A, uint32_t B, uint32_t C, void* st) {
    if (A == 0 || B == 0 || C == 0) return 0;
    ZK_ARG(out != in && out != nullptr && in != nullptr, "zk_fr_swap_axes: null or in-place");
    ZK_ARG((size_t)A * B <= 0x7FFFFFFFull && C <= 0x7FFFFFFFu, "zk_fr_swap_axes: too many rows for one launch");
    hipLaunchKernelGGL(k_swap_axes, dim3(A * B), dim3(TPB), 0, (hipStream_t)st, (uint4*)out, (const uint4*)in, A, B, C * 2);
    ZK_LAUNCH_CHECK();
    return 0;
}
// dst[i] = src[offset + i * stride] for elements of `words` 16-byte words (a field element 2, a Jacobian point 9)
__global__ void __launch_bounds__(TPB) k_copy_strided(uint4* __restrict__ dst, const uint4* __restrict__ src, uint32_t words, size_t count, size_t stride, size_t offset) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= count * words) return;
    const size_t e = i / words, w = i - e * words;
    dst[i] = src[(offset + e * stride) * words + w];
}
int zk_copy_strided(void* dst, const void* src, size_t elem_bytes, size_t count, size_t stride, size_t offset, void* st) {
    ZK_ARG(elem_bytes >= 16 && elem_bytes % 16 == 0 && elem_bytes <= 1024, "zk_copy_strided: elements of 16 to 1024 bytes, a multiple of 16");
    ZK_ARG(dst != src, "zk_copy_strided: in place");
    if (count == 0) return 0;
    const uint32_t words = (uint32_t)(elem_bytes / 16);
    LAUNCH1D(k_copy_strided, count * words, st, (uint4*)dst, (const uint4*)src, words, count, stride, offset);
    return 0;
}
int zk_fr_gather(void* out, const void* table, const void* idx, size_t n, void* st) {
    LAUNCH1D(k_gather, n, st, (Fr*)out, (const Fr*)table, (const uint32_t*)idx, n);
    return 0;
}

int zk_fr_sum(uint32_t* out_host, const void* a, size_t n, void* st) {
    if (n == 0) { memset(out_host, 0, 32); return 0; }
    const unsigned nb = reduce_grid(n);
    Scratch part(sizeof(Fr) * nb, (hipStream_t)st);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_sum, dim3(nb), dim3(TPB), 0, (hipStream_t)st, part.as<Fr>(), (const Fr*)a, n);
    ZK_LAUNCH_CHECK();
    return finish_to_host<1>(part.as<Fr>(), nb, (Fr*)out_host, (hipStream_t)st);
}
// sum_i a_i * b_i in standard form
int zk_fr_dot(uint32_t* out_host, const void* a, const void* b, size_t n, void* st) {
    if (n == 0) { memset(out_host, 0, 32); return 0; }
    const unsigned nb = reduce_grid(n);
    Scratch part(sizeof(Fr) * nb, (hipStream_t)st);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_dot, dim3(nb), dim3(TPB), 0, (hipStream_t)st, part.as<Fr>(), (const Fr*)a, (const Fr*)b, n);
    ZK_LAUNCH_CHECK();
    Fr s;
    int rc = finish_to_host<1>(part.as<Fr>(), nb, &s, (hipStream_t)st);
    if (rc) return rc;
    s = to_mont(s);
    memcpy(out_host, &s, 32);
    return 0;
}

// One or more levels of the middle-axis fold; u[0..levels) are standard-form challenges.
// out has other * ceil(cur / 2^levels) * window elements.  levels <= 3 per call.
int zk_fr_fold_axis(void* out, const void* in, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* st) {
    ZK_ARG(levels >= 1 && levels <= 3, "zk_fr_fold_axis: levels must be 1..3");
    ZK_ARG(cur >= 1 && window >= 1, "zk_fr_fold_axis: empty axis");
    ZK_ARG(out != in, "zk_fr_fold_axis: out must differ from in");
    const uint32_t cur_out = (uint32_t)(((uint64_t)cur + (1u << levels) - 1) >> levels);
    const size_t n_out = other * cur_out * window;
    if (n_out == 0) return 0;
    if (levels == 1) {
        FrPack<1> p; p.x[0] = to_mont(load_fr(u));
        LAUNCH1D(k_fold_axis<1>, n_out, st, (Fr*)out, (const Fr*)in, p, n_out, cur, cur_out, window);
    } else {
        // weights of the 2^levels inputs of one output, Montgomery form
        Fr x[3], w[8];
        for (int i = 0; i < levels; ++i) x[i] = to_mont(load_fr(u + 8 * i));
        const Fr one = big_one_mont<8>();
        for (int j = 0; j < (1 << levels); ++j) {
            Fr p = (j & 1) ? x[0] : sub(one, x[0]);
            for (int l = 1; l < levels; ++l) p = mont_mul(p, ((j >> l) & 1) ? x[l] : sub(one, x[l]));
            w[j] = p;
        }
        if (levels == 2) {
            FrPack<4> p; for (int j = 0; j < 4; ++j) p.x[j] = w[j];
            LAUNCH1D(k_fold_axis_dot<2>, n_out, st, (Fr*)out, (const Fr*)in, p, n_out, cur, cur_out, window);
        } else {
            FrPack<8> p; for (int j = 0; j < 8; ++j) p.x[j] = w[j];
            LAUNCH1D(k_fold_axis_dot<3>, n_out, st, (Fr*)out, (const Fr*)in, p, n_out, cur, cur_out, window);
        }
    }
    return 0;
}

// Multilinear extension of a (n elements, zero-extended to 2^k) at u[0..k): index bit j is bound
// to u[j].  Requires 2^(k-1) < n <= 2^k (k = 0 allowed for n == 1).
int zk_fr_me(uint32_t* out_host, const void* a, size_t n, const uint32_t* u, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(n >= 1 && k >= 0 && k <= 32, "zk_fr_me: bad size");
    ZK_ARG(n <= ((size_t)1 << k) && (k == 0 || n > ((size_t)1 << (k - 1))), "zk_fr_me: need 2^(k-1) < n <= 2^k");
    const Fr* cur_ptr = (const Fr*)a;
    size_t cur = n;
    int done = 0;
    void* bufs[2] = {nullptr, nullptr};
    int which = 0, rc = 0;
    while (cur > ME_SMALL_MAX && rc == 0) {
        const int L = 3;
        const size_t next = (cur + 7) >> 3;
        if (!bufs[which]) rc = pool_alloc(&bufs[which], next * sizeof(Fr), st);
        if (rc) break;
        rc = zk_fr_fold_axis(bufs[which], cur_ptr, u + 8 * done, L, 1, (uint32_t)cur, 1, stv);
        cur_ptr = (const Fr*)bufs[which];
        which ^= 1;
        cur = next;
        done += L;
    }
    if (rc == 0) {
        FrPack12 p;
        const int rest = k - done;
        for (int i = 0; i < 12; ++i) p.x[i] = (i < rest) ? to_mont(load_fr(u + 8 * (done + i))) : big_zero<8>();
        Scratch fin(sizeof(Fr), st);
        rc = fin.rc;
        if (!rc) {
            hipLaunchKernelGGL(k_me_small, dim3(1), dim3(TPB), 0, st, fin.as<Fr>(), cur_ptr, p, (uint32_t)cur, (uint32_t)rest);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = hip_fail(e, "zk_fr_me", __FILE__, __LINE__);
            else rc = deliver(st, fin.p, out_host, 1, 0);
        }
    }
    for (int i = 0; i < 2; ++i) if (bufs[i]) pool_free(bufs[i], st);
    return rc;
}

int zk_fr_fold_halves(void* out, const void* a, const uint32_t* v, size_t n_in, size_t n_out, void* st) {
    ZK_ARG(out != a, "zk_fr_fold_halves: out must differ from in");
    LAUNCH1D(k_fold_halves, n_out, st, (Fr*)out, (const Fr*)a, to_mont(load_fr(v)), n_in, n_out);
    return 0;
}

// One round of the inner-product sumcheck: poly3_host = [sum a0 b0, sum a0 db + b0 da, sum da db].
int zk_ip_round(uint32_t* poly3_host, const void* a, const void* b, size_t n_in, size_t n_out, void* stv) {
    ZK_ARG(n_out >= 1 && n_in >= 1 && n_in <= 2 * n_out, "zk_ip_round: need n_in <= 2*n_out");
    const unsigned nb = reduce_grid(n_out);
    Scratch part(sizeof(Fr) * 3 * nb, (hipStream_t)stv);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_ip_round, dim3(nb), dim3(TPB), 0, (hipStream_t)stv, part.as<Fr>(), (const Fr*)a, (const Fr*)b, n_in, n_out);
    ZK_LAUNCH_CHECK();
    Scratch fin(sizeof(Fr) * 3, (hipStream_t)stv);
    if (fin.rc) return fin.rc;
    hipLaunchKernelGGL(k_finish_sums, dim3(3), dim3(TPB), 0, (hipStream_t)stv, fin.as<Fr>(), part.as<Fr>(), nb);
    ZK_LAUNCH_CHECK();
    return deliver((hipStream_t)stv, fin.p, poly3_host, 3, 3);
}

// Stacked round over [N][D] tensors: rows_in = N, rows_out = 2^ceil(log2 N) / 2, E = eq table over the
// remaining stacking challenges (rows_out entries, Montgomery form).
int zk_ip_round_stacked(uint32_t* poly3_host, const void* a, const void* b, const void* E, size_t D, size_t rows_in, size_t rows_out, void* stv) {
    ZK_ARG(D >= 1 && rows_out >= 1 && rows_in >= 1 && rows_in <= 2 * rows_out, "zk_ip_round_stacked: bad shape");
    const size_t n_in = rows_in * D, n_out = rows_out * D;
    const unsigned nb = reduce_grid(n_out);
    Scratch part(sizeof(Fr) * 3 * nb, (hipStream_t)stv);
    if (part.rc) return part.rc;
    hipLaunchKernelGGL(k_ip_round_w, dim3(nb), dim3(TPB), 0, (hipStream_t)stv, part.as<Fr>(), (const Fr*)a, (const Fr*)b, (const Fr*)E, D, n_in, n_out);
    ZK_LAUNCH_CHECK();
    Fr s[3];
    int rc = finish_to_host<3>(part.as<Fr>(), nb, s, (hipStream_t)stv);
    if (rc) return rc;
    for (int i = 0; i < 3; ++i) s[i] = to_mont(s[i]);
    memcpy(poly3_host, s, 96);
    return 0;
}

// Complete inner-product sumcheck for n <= 8192 in one launch.  u[0..k) standard form, consumed
// from the back; polys_host gets 3*k coefficients, fin_host the folded a and b.
int zk_ip_sumcheck_small(uint32_t* polys_host, uint32_t* fin_host, const void* a, const void* b, uint32_t n, const uint32_t* u, int k, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(k >= 1 && k <= 13, "zk_ip_sumcheck_small: k must be 1..13");
    ZK_ARG(n >= 1 && n <= (1u << k) && n > ((1u << k) >> 1), "zk_ip_sumcheck_small: need 2^(k-1) < n <= 2^k");
    FrPack16 p;
    for (int i = 0; i < 16; ++i) p.x[i] = (i < k) ? to_mont(load_fr(u + 8 * i)) : big_zero<8>();
    const size_t half0 = ((size_t)1 << k) >> 1;
    Scratch work(sizeof(Fr) * (4 * half0 + 3 * (size_t)k + 2), st);
    if (work.rc) return work.rc;
    Fr* w = work.as<Fr>();
    Fr* polys = w + 4 * half0;
    Fr* fin = polys + 3 * k;
    hipLaunchKernelGGL(k_ip_small, dim3(1), dim3(1024), 0, st, polys, fin, w, (const Fr*)a, (const Fr*)b, p, n, (uint32_t)k);
    ZK_LAUNCH_CHECK();
    // one delivery of 3k + 2 values: the round polynomials, then the two fully folded values
    Fr both[3 * 13 + 2];
    int rc = deliver(st, polys, both, 3 * (size_t)k + 2, 0);
    if (rc) return rc;
    memcpy(polys_host, both, sizeof(Fr) * 3 * k);           // (while results are deferred these two are not what the kernel wrote: see zk_defer_begin)
    memcpy(fin_host, both + 3 * k, sizeof(Fr) * 2);
    return 0;
}

int zk_fr_sum_static(void* out_dev, const void* a, size_t n, void* st) {
    ZK_ARG(out_dev != nullptr, "zk_fr_sum_static: null output");
    ZK_ARG(n <= ZK_FR_SUM_STATIC_MAX_N, "zk_fr_sum_static: more than 2^32 - 1 elements (ZK_FR_SUM_STATIC_MAX_N)");
    ZK_ARG(n == 0 || a != nullptr, "zk_fr_sum_static: null input");
    Fr* part = nullptr;
    int rc = scratch_address(&part);
    if (rc) return rc;
    const unsigned nb = n ? reduce_grid(n) : 1;       // n == 0: one block that writes a zero partial
    hipLaunchKernelGGL(k_sum, dim3(nb), dim3(TPB), 0, (hipStream_t)st, part, (const Fr*)a, n);
    ZK_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_finish_sums, dim3(1), dim3(TPB), 0, (hipStream_t)st, (Fr*)out_dev, (const Fr*)part, nb);
    ZK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

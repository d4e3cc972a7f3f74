// Fr matrix product C[M x P] = A[M x N] * B[N x P] for gfx950 (replaces matrixMultiplyOptimized,
// fr-tensor.cu:831-881, used by zkFC::operator() zkfc.cu:44-58 and FrTensor::matmul).
//
// The work is VALU integer multiply-add (v_mad_u64_u32); MFMA cannot help a 255-bit modular
// product.  Two paths, both bit-identical to the reference because results are canonical:
//
//  * generic: every MAC is a 255x255-bit product.  Eight products are accumulated limb-row by
//    column by column into one running value and share a single Montgomery reduction: 64
//    multiply-adds per MAC for the products plus 64/8 for the reduction, against 128 for a
//    product reduced on its own.  The R^-1 factor is removed once per output.
//  * small-integer: when both operands are embeddings of int32-range values and the whole dot
//    product is bounded by 2^62, the same sum is computed in int64 and embedded at the end.
//    The bound is established on the device from the operands (largest row sum of |a| times max |b|);
//    nothing is assumed.  This is the case for every matmul of the LLaMa pipeline except softmax(Y)*V.
//    Large products of this kind (the seven projections of a layer) are plain integer GEMMs and go to the matrix
//    cores: both operands are split into balanced base-256 digits (int8 planes), every pair of planes is an int8 GEMM
//    with int32 accumulation (k_gemm_i8_planes_all: v_mfma_i32_32x32x32_i8 tiles), planes of equal weight 2^(8s) accumulate into the same output, and one
//    pass recombines the outputs in int64.  Exact: a dot product of digits stays below 2^31 (checked), the
//    recombined value is the true integer result, below 2^62 by the bound above.
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>
#include "field.hpp"
#include "rt.hpp"
#include "../../include/zkllm_hip.h"

using namespace zk;

static constexpr int KT = 8;       // terms sharing one reduction
static constexpr int TM = 16, TN = 16;

// sum_q a[q]*b[q]*R^-1 mod r, canonical.  Product scanning: column k gathers the limb products of all KT
// terms and of the reduction in one 96-bit accumulator (at most 72 products of 64 bits per column), so a
// limb product costs one multiply-add and one add-with-carry.  The value before the final subtractions is
// below (KT*r/R + 1)*r < 5r.
__device__ __forceinline__ Fr dot_mont(const Fr (&a)[KT], const Fr (&b)[KT]) {
    uint32_t m[8], t[9];
    uint64_t lo = 0;
    uint32_t hi = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#pragma unroll
        for (int q = 0; q < KT; q += 4) {
#pragma unroll
            for (int i = 0; i <= k; ++i)
                mac96v4(lo, hi, a[q].v[i], b[q].v[k - i], a[q + 1].v[i], b[q + 1].v[k - i], a[q + 2].v[i], b[q + 2].v[k - i], a[q + 3].v[i], b[q + 3].v[k - i]);
        }
        {
            uint32_t pr[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) pr[i] = FrK::P((k - i) & 7);
            if (k == 1) mac_chain<1, true>(lo, hi, m, pr);
            if (k == 2) mac_chain<2, true>(lo, hi, m, pr);
            if (k == 3) mac_chain<3, true>(lo, hi, m, pr);
            if (k == 4) mac_chain<4, true>(lo, hi, m, pr);
            if (k == 5) mac_chain<5, true>(lo, hi, m, pr);
            if (k == 6) mac_chain<6, true>(lo, hi, m, pr);
            if (k == 7) mac_chain<7, true>(lo, hi, m, pr);
        }
        m[k] = 0u - (uint32_t)lo;                     // INV = -1 mod 2^32
        col_shift_reduce<FrK::P(0)>(lo, hi, m[k]);
    }
#pragma unroll
    for (int k = 8; k < 16; ++k) {
#pragma unroll
        for (int q = 0; q < KT; q += 4) {
#pragma unroll
            for (int i = k - 7; i < 8; ++i)
                mac96v4(lo, hi, a[q].v[i], b[q].v[k - i], a[q + 1].v[i], b[q + 1].v[k - i], a[q + 2].v[i], b[q + 2].v[k - i], a[q + 3].v[i], b[q + 3].v[k - i]);
        }
        {
            uint32_t pr[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) pr[i] = FrK::P((7 - i) & 7);     // m[k-7+i] pairs with P(7-i)
            if (k == 8) mac_chain<7, true>(lo, hi, m + 1, pr);
            if (k == 9) mac_chain<6, true>(lo, hi, m + 2, pr);
            if (k == 10) mac_chain<5, true>(lo, hi, m + 3, pr);
            if (k == 11) mac_chain<4, true>(lo, hi, m + 4, pr);
            if (k == 12) mac_chain<3, true>(lo, hi, m + 5, pr);
            if (k == 13) mac_chain<2, true>(lo, hi, m + 6, pr);
            if (k == 14) mac_chain<1, true>(lo, hi, m + 7, pr);
        }
        t[k - 8] = (uint32_t)lo;
        lo = (lo >> 32) | ((uint64_t)hi << 32);
        hi = 0;
    }
    t[8] = (uint32_t)lo;
    // t[0..8] < (KT+1) r : subtract 8r, 4r, 2r, r conditionally (constants built at compile time)
#pragma unroll
    for (int s = 3; s >= 0; --s) {
        uint32_t d[9];
        uint64_t br = 0;
#pragma unroll
        for (int i = 0; i < 9; ++i) {
            // limb i of (r << s)
            const uint32_t lo = (i < 8) ? FrK::P(i) : 0u;
            const uint32_t prev = (i >= 1 && i <= 8) ? FrK::P(i - 1) : 0u;
            const uint32_t ki = (s == 0) ? lo : (uint32_t)((lo << s) | (prev >> (32 - s)));
            uint64_t x = (uint64_t)t[i] - ki - br;
            d[i] = (uint32_t)x;
            br = (x >> 32) & 1u;
        }
        const bool keep = br != 0;
#pragma unroll
        for (int i = 0; i < 9; ++i) t[i] = keep ? t[i] : d[i];
    }
    Fr r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = t[i];
    return r;
}

__global__ void __launch_bounds__(TM * TN) k_matmul(Fr* __restrict__ C, const Fr* __restrict__ A, const Fr* __restrict__ B, uint32_t M, uint32_t N, uint32_t P) {
    __shared__ uint32_t As[8][TM][KT + 1];
    __shared__ uint32_t Bs[8][KT][TN];
    A += (size_t)blockIdx.z * M * N; B += (size_t)blockIdx.z * N * P; C += (size_t)blockIdx.z * M * P;   // one product of a stack per grid plane
    const uint32_t tx = threadIdx.x % TN, ty = threadIdx.x / TN;
    const uint32_t row = blockIdx.y * TM + ty, col = blockIdx.x * TN + tx;
    Fr acc = big_zero<8>();
    for (uint32_t k0 = 0; k0 < N; k0 += KT) {
        // 128 A elements + 128 B elements, one per thread
        if (threadIdx.x < TM * KT) {
            const uint32_t r = threadIdx.x / KT, q = threadIdx.x % KT;
            const uint32_t gr = blockIdx.y * TM + r, gk = k0 + q;
            Fr v = (gr < M && gk < N) ? A[(size_t)gr * N + gk] : big_zero<8>();
#pragma unroll
            for (int l = 0; l < 8; ++l) As[l][r][q] = v.v[l];
        } else {
            const uint32_t e = threadIdx.x - TM * KT;
            const uint32_t q = e / TN, c = e % TN;
            const uint32_t gk = k0 + q, gc = blockIdx.x * TN + c;
            Fr v = (gk < N && gc < P) ? B[(size_t)gk * P + gc] : big_zero<8>();
#pragma unroll
            for (int l = 0; l < 8; ++l) Bs[l][q][c] = v.v[l];
        }
        __syncthreads();
        Fr a[KT], b[KT];
#pragma unroll
        for (int q = 0; q < KT; ++q) {
#pragma unroll
            for (int l = 0; l < 8; ++l) { a[q].v[l] = As[l][ty][q]; b[q].v[l] = Bs[l][q][tx]; }
        }
        acc = add(acc, dot_mont(a, b));
        __syncthreads();
    }
    if (row < M && col < P) C[(size_t)row * P + col] = to_mont(acc);
}

// ---- small-integer path ---------------------------------------------------------------------------
// max |x| over a tensor of embedded integers; anything that is not an embedded int64 in
// [-2^62, 2^62] poisons the result with UINT64_MAX.
__global__ void __launch_bounds__(256) k_absmax(unsigned long long* __restrict__ out, const Fr* __restrict__ a, size_t n) {
    unsigned long long m = 0;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const Fr x = a[i];
        unsigned long long v;
        if (!(x.v[2] | x.v[3] | x.v[4] | x.v[5] | x.v[6] | x.v[7])) v = (unsigned long long)x.v[0] | ((unsigned long long)x.v[1] << 32);
        else {
            const Fr y = neg(x);
            v = (y.v[2] | y.v[3] | y.v[4] | y.v[5] | y.v[6] | y.v[7]) ? ~0ull : ((unsigned long long)y.v[0] | ((unsigned long long)y.v[1] << 32));
        }
        if (v > (1ull << 62)) v = ~0ull;
        m = v > m ? v : m;
    }
    __shared__ unsigned long long red[256];
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] = red[threadIdx.x] > red[threadIdx.x + s] ? red[threadIdx.x] : red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) atomicMax(out, red[0]);
}
// max over rows of sum_j |a[row][j]| (saturating): with max |b| it bounds every dot product more tightly than
// N * max|a| * max|b| does -- rows of a softmax output sum to its scale however long they are.
// The same pass takes the largest magnitude of the tensor (out_max, as k_absmax delivers it) along.
__global__ void __launch_bounds__(256) k_rowabs(unsigned long long* __restrict__ out, unsigned long long* __restrict__ out_max, const Fr* __restrict__ a, uint32_t ncol) {
    const Fr* row = a + (size_t)blockIdx.x * ncol;
    unsigned long long m = 0, mx = 0;
    for (uint32_t j = threadIdx.x; j < ncol; j += 256) {
        const Fr x = row[j];
        unsigned long long v;
        if (!(x.v[2] | x.v[3] | x.v[4] | x.v[5] | x.v[6] | x.v[7])) v = (unsigned long long)x.v[0] | ((unsigned long long)x.v[1] << 32);
        else {
            const Fr y = neg(x);
            v = (y.v[2] | y.v[3] | y.v[4] | y.v[5] | y.v[6] | y.v[7]) ? ~0ull : ((unsigned long long)y.v[0] | ((unsigned long long)y.v[1] << 32));
        }
        if (v > (1ull << 62)) v = ~0ull;
        mx = v > mx ? v : mx;
        m = (m == ~0ull || v == ~0ull || m + v > (1ull << 62)) ? ~0ull : m + v;
    }
    // both figures through one tree: wave shuffles first, one LDS step for the four waves
    auto sat_add = [](unsigned long long x, unsigned long long y) { return (x == ~0ull || y == ~0ull || x + y > (1ull << 62)) ? ~0ull : x + y; };
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long om = __shfl_xor(mx, off, 64), os = __shfl_xor(m, off, 64);
        mx = om > mx ? om : mx;
        m = sat_add(m, os);
    }
    __shared__ unsigned long long red[2][4];
    const uint32_t wv = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0) { red[0][wv] = mx; red[1][wv] = m; }
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long gm = red[0][0], gs = red[1][0];
        for (int i = 1; i < 4; ++i) { gm = red[0][i] > gm ? red[0][i] : gm; gs = sat_add(gs, red[1][i]); }
        // a row that raises neither figure leaves them alone: with one workgroup per row, tens of thousands of atomics on
        // the same two words are what the launch would otherwise wait for (the figures only grow, so a stale read costs an
        // atomic that changes nothing and never drops one that would)
        if (gm > __atomic_load_n(out_max, __ATOMIC_RELAXED)) atomicMax(out_max, gm);
        if (gs > __atomic_load_n(out, __ATOMIC_RELAXED)) atomicMax(out, gs);
    }
}
// A left operand that exists as the elementwise product of two tensors in int32 form (a softmax's output: the product of two
// segments' table values): its elements are exact 64-bit integers, read at 8 bytes each instead of 32.
// b null: the operand is a itself, a tensor read from its int32 form.
struct ProdSrc { const int32_t* a; const int32_t* b; };
__device__ __forceinline__ long long prod_at(const ProdSrc& s, size_t i) { return s.b ? (long long)s.a[i] * (long long)s.b[i] : (long long)s.a[i]; }
// k_rowabs for such an operand
__global__ void __launch_bounds__(256) k_rowabs_prod(unsigned long long* __restrict__ out, unsigned long long* __restrict__ out_max, const ProdSrc src, uint32_t ncol) {
    const size_t base = (size_t)blockIdx.x * ncol;
    unsigned long long m = 0, mx = 0;
    for (uint32_t j = threadIdx.x; j < ncol; j += 256) {
        const long long x = prod_at(src, base + j);
        unsigned long long v = x < 0 ? 0ull - (unsigned long long)x : (unsigned long long)x;
        if (v > (1ull << 62)) v = ~0ull;
        mx = v > mx ? v : mx;
        m = (m == ~0ull || v == ~0ull || m + v > (1ull << 62)) ? ~0ull : m + v;
    }
    auto sat_add = [](unsigned long long x, unsigned long long y) { return (x == ~0ull || y == ~0ull || x + y > (1ull << 62)) ? ~0ull : x + y; };
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long om = __shfl_xor(mx, off, 64), os = __shfl_xor(m, off, 64);
        mx = om > mx ? om : mx;
        m = sat_add(m, os);
    }
    __shared__ unsigned long long red[2][4];
    const uint32_t wv = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0) { red[0][wv] = mx; red[1][wv] = m; }
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long gm = red[0][0], gs = red[1][0];
        for (int i = 1; i < 4; ++i) { gm = red[0][i] > gm ? red[0][i] : gm; gs = sat_add(gs, red[1][i]); }
        if (gm > __atomic_load_n(out_max, __ATOMIC_RELAXED)) atomicMax(out_max, gm);
        if (gs > __atomic_load_n(out, __ATOMIC_RELAXED)) atomicMax(out, gs);
    }
}
// the operand written out as field elements (for the paths that read nothing else)
__global__ void __launch_bounds__(256) k_prod_to_fr(Fr* __restrict__ out, const ProdSrc src, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = fr_from_i64(prod_at(src, i));
}
template <typename T> __global__ void __launch_bounds__(256) k_fr_to_int(T* __restrict__ out, const Fr* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (T)fr_to_i64(a[i]);
}
// 64x64 output tile per workgroup, 4x4 per thread, K step 16, int64 accumulation.
// T = int when both operands fit 31 bits (one v_mad_i64_i32 per MAC), long long otherwise.
template <typename T> __global__ void __launch_bounds__(256) k_matmul_int(Fr* __restrict__ C, const T* __restrict__ A, const T* __restrict__ B, uint32_t M, uint32_t N, uint32_t P) {
    __shared__ T As[16][64 + 1];
    __shared__ T Bs[16][64 + 1];
    A += (size_t)blockIdx.z * M * N; B += (size_t)blockIdx.z * N * P; C += (size_t)blockIdx.z * M * P;   // one product of a stack per grid plane
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const uint32_t row0 = blockIdx.y * 64, col0 = blockIdx.x * 64;
    long long acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0;
    for (uint32_t k0 = 0; k0 < N; k0 += 16) {
        for (uint32_t e = threadIdx.x; e < 64 * 16; e += 256) {
            const uint32_t r = e / 16, q = e % 16;        // A: 64 rows x 16 k
            As[q][r] = (row0 + r < M && k0 + q < N) ? A[(size_t)(row0 + r) * N + k0 + q] : (T)0;
            const uint32_t q2 = e / 64, c = e % 64;       // B: 16 k x 64 cols
            Bs[q2][c] = (k0 + q2 < N && col0 + c < P) ? B[(size_t)(k0 + q2) * P + col0 + c] : (T)0;
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            T av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[q][ty * 4 + i]; bv[i] = Bs[q][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += (long long)av[i] * (long long)bv[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = row0 + ty * 4 + i, c = col0 + tx * 4 + j;
            if (r < M && c < P) C[(size_t)r * P + c] = fr_from_i64(acc[i][j]);
        }
}

// The same tiling for a wide left operand (|a| < 2^62) and a right operand that fits 31 bits: a = hi * 2^31 + lo with
// 0 <= lo < 2^31, and each half takes one v_mad_i64_i32 per product; the two sums are recombined modulo 2^64, which is exact
// because the true result is below 2^62 in magnitude.  Two multiply-adds per product instead of a 64 x 64-bit product.
__global__ void __launch_bounds__(256) k_matmul_wide_narrow(Fr* __restrict__ C, const long long* __restrict__ A, const int* __restrict__ B, uint32_t M, uint32_t N, uint32_t P) {
    __shared__ int Alo[16][64 + 1];
    __shared__ int Ahi[16][64 + 1];
    __shared__ int Bs[16][64 + 1];
    A += (size_t)blockIdx.z * M * N; B += (size_t)blockIdx.z * N * P; C += (size_t)blockIdx.z * M * P;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const uint32_t row0 = blockIdx.y * 64, col0 = blockIdx.x * 64;
    long long lo[4][4], hi[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) { lo[i][j] = 0; hi[i][j] = 0; }
    for (uint32_t k0 = 0; k0 < N; k0 += 16) {
        for (uint32_t e = threadIdx.x; e < 64 * 16; e += 256) {
            const uint32_t r = e / 16, q = e % 16;        // A: 64 rows x 16 k
            const long long a = (row0 + r < M && k0 + q < N) ? A[(size_t)(row0 + r) * N + k0 + q] : 0ll;
            Alo[q][r] = (int)(a & 0x7FFFFFFFll);
            Ahi[q][r] = (int)(a >> 31);
            const uint32_t q2 = e / 64, c = e % 64;       // B: 16 k x 64 cols
            Bs[q2][c] = (k0 + q2 < N && col0 + c < P) ? B[(size_t)(k0 + q2) * P + col0 + c] : 0;
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            int al[4], ah[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { al[i] = Alo[q][ty * 4 + i]; ah[i] = Ahi[q][ty * 4 + i]; bv[i] = Bs[q][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    lo[i][j] += (long long)al[i] * (long long)bv[j];
                    hi[i][j] += (long long)ah[i] * (long long)bv[j];
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = row0 + ty * 4 + i, c = col0 + tx * 4 + j;
            const long long v = (long long)(((unsigned long long)hi[i][j] << 31) + (unsigned long long)lo[i][j]);
            if (r < M && c < P) C[(size_t)r * P + c] = fr_from_i64(v);
        }
}
static int run_wide_narrow_path(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, hipStream_t st) {
    const size_t na = (size_t)batch * M * N, nb = (size_t)batch * N * P;
    Scratch ai(na * sizeof(long long), st), bi(nb * sizeof(int), st);
    if (ai.rc) return ai.rc;
    if (bi.rc) return bi.rc;
    hipLaunchKernelGGL(k_fr_to_int<long long>, dim3(cdiv(na, 256)), dim3(256), 0, st, ai.as<long long>(), (const Fr*)A, na);
    hipLaunchKernelGGL(k_fr_to_int<int>, dim3(cdiv(nb, 256)), dim3(256), 0, st, bi.as<int>(), (const Fr*)B, nb);
    hipLaunchKernelGGL(k_matmul_wide_narrow, dim3(cdiv(P, 64), cdiv(M, 64), batch), dim3(256), 0, st, (Fr*)C, ai.as<long long>(), bi.as<int>(), M, N, P);
    ZK_LAUNCH_CHECK();
    return 0;
}

template <typename T> static int run_int_path(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, hipStream_t st) {
    const size_t na = (size_t)batch * M * N, nb = (size_t)batch * N * P;
    Scratch ai(na * sizeof(T), st), bi(nb * sizeof(T), st);
    if (ai.rc) return ai.rc;
    if (bi.rc) return bi.rc;
    hipLaunchKernelGGL(k_fr_to_int<T>, dim3(cdiv(na, 256)), dim3(256), 0, st, ai.as<T>(), (const Fr*)A, na);
    hipLaunchKernelGGL(k_fr_to_int<T>, dim3(cdiv(nb, 256)), dim3(256), 0, st, bi.as<T>(), (const Fr*)B, nb);
    hipLaunchKernelGGL(k_matmul_int<T>, dim3(cdiv(P, 64), cdiv(M, 64), batch), dim3(256), 0, st, (Fr*)C, ai.as<T>(), bi.as<T>(), M, N, P);
    ZK_LAUNCH_CHECK();
    return 0;
}

// ---- int8-plane path: digit planes and a GEMM on the matrix cores ------------------------------------------------------
// Balanced base-256 digits of a small signed integer: x = sum_j d_j 256^j, d_j in [-128, 127].  Both operands are laid
// out with the contraction index fastest and padded with zeros to a multiple of the GEMM's K tile:
//   planes of A[b][m][k]:  PA[((b * pa + i) * M + m) * Kp + k]
//   planes of B[b][k][p]:  PB[((b * pb + j) * P + p) * Kp + k]      (transposed on the way)
// so that every operand fragment of the matrix instruction is 16 consecutive bytes.
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
static constexpr int GBM = 128, GBN = 128, GBK = 128;      // block tile of the GEMM: 4 waves, 64 x 64 outputs each
static constexpr int GLD = GBK + 16;                       // LDS row stride in bytes: 16-byte aligned rows whose 16-byte reads spread over all banks

// src: the operand as a product of int32 forms when src.a is set (a is then not read)
__global__ void __launch_bounds__(256) k_split_rows(int8_t* __restrict__ planes, const Fr* __restrict__ a, const ProdSrc src, size_t rows, uint32_t M, uint32_t N, uint32_t Kp, int np) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const uint32_t groups = Kp / 4;
    // 32-bit divisions where the launch has fewer than 2^32 lanes (the same for every lane; rows is below 2^31): a 64-bit
    // division costs more than forming a plane's four digits
    size_t row;
    uint32_t k;
    if (rows * (size_t)groups <= 0xFFFFFFFFull) {
        const uint32_t g32 = (uint32_t)gid, r32 = g32 / groups;
        row = r32;
        k = 4 * (g32 - r32 * groups);
    } else {
        row = gid / groups;
        k = 4 * (uint32_t)(gid % groups);
    }
    if (row >= rows) return;
    const uint32_t b32 = (uint32_t)row / M;
    const size_t b = b32, m = (uint32_t)row - b32 * M;
    long long x[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = (k + e < N) ? (src.a ? prod_at(src, row * N + k + e) : fr_to_i64(a[row * N + k + e])) : 0ll;
    for (int j = 0; j < np; ++j) {
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const long long d = (long long)(int8_t)(x[e] & 0xFF);
            x[e] = (x[e] - d) >> 8;
            packed |= (uint32_t)(uint8_t)d << (8 * e);
        }
        *reinterpret_cast<uint32_t*>(planes + ((b * np + j) * M + m) * Kp + k) = packed;
    }
}
// grid (P tiles of 64, K tiles of 64, batch): a 64 x 64 tile of B goes through LDS so that reads run along p and writes along k
__global__ void __launch_bounds__(256) k_split_cols(int8_t* __restrict__ planes, const Fr* __restrict__ B, uint32_t N, uint32_t P, uint32_t Kp, int np) {
    __shared__ __attribute__((aligned(16))) int8_t tile[8][64][80];
    const uint32_t t = threadIdx.x, p = t & 63, kq = t >> 6;
    const uint32_t p0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
    const size_t b = blockIdx.z;
    for (int r = 0; r < 16; ++r) {
        const uint32_t k = k0 + kq * 16 + r;
        long long x = (k < N && p0 + p < P) ? fr_to_i64(B[(b * N + k) * P + p0 + p]) : 0ll;
        for (int j = 0; j < np; ++j) {
            const long long d = (long long)(int8_t)(x & 0xFF);
            x = (x - d) >> 8;
            tile[j][p][kq * 16 + r] = (int8_t)d;
        }
    }
    __syncthreads();
    const uint32_t row = t >> 2, ch = t & 3;
    if (p0 + row < P)
        for (int j = 0; j < np; ++j)
            *reinterpret_cast<v4i*>(planes + ((b * np + j) * P + p0 + row) * Kp + k0 + ch * 16) = *reinterpret_cast<const v4i*>(&tile[j][row][ch * 16]);
}

// C[b][m][p] = sum_{i,j} 256^(i+j) sum_k PA_i[b][m][k] PB_j[b][p][k], embedded in Fr.
// One block computes a 128 x 128 tile of C; each of its four waves a 64 x 64 quarter as 2 x 2 tiles of
// v_mfma_i32_32x32x32_i8.  Plane pairs are taken one after the other: int32 accumulators over the whole contraction
// (|sum| <= K * 2^14, the caller keeps K below 2^17), then shifted into the int64 totals, which are exact modulo 2^64 and
// therefore exact, the true result being below 2^62.  Operand tiles of 128 rows x 128 bytes pass through LDS; the next
// tile is fetched into registers while the current one is multiplied.
// Fragments: lane l supplies row (or column) l % 32 and the 16 contraction bytes 16 (l / 32) + 0..15 of a 32-byte step for
// both operands alike, so whatever order the instruction takes the bytes in, every product pairs equal k.  Outputs:
// register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of the 32 x 32 tile.
// C64 set: the products are written there as 64-bit integers (8 bytes an element) and C is not written
struct PlaneGemm { const int8_t* A; const int8_t* B; Fr* C; uint32_t M, P, Kp; int pa, pb; long long* C64; };
__device__ __forceinline__ void gemm_store(const PlaneGemm& g, size_t at, long long v) {
    if (g.C64) g.C64[at] = v;
    else g.C[at] = fr_from_i64(v);
}
__global__ void __launch_bounds__(256) k_gemm_i8_planes(const PlaneGemm g) {
    __shared__ __attribute__((aligned(16))) int8_t sA[GBM * GLD];
    __shared__ __attribute__((aligned(16))) int8_t sB[GBN * GLD];
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
    const uint32_t m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;
    const size_t b = blockIdx.z;
    long long tot[4][16];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) tot[q][r] = 0;
    for (int i = 0; i < g.pa; ++i)
        for (int j = 0; j < g.pb; ++j) {
            const int8_t* __restrict__ Ai = g.A + ((b * g.pa + i) * g.M) * (size_t)g.Kp;
            const int8_t* __restrict__ Bj = g.B + ((b * g.pb + j) * g.P) * (size_t)g.Kp;
            v16i acc[4];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[q][r] = 0;
            v4i ra[4], rb[4];
            auto fetch = [&](uint32_t k0) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t c = t + 256 * q, row = c >> 3, kc = c & 7;
                    const v4i zero = {0, 0, 0, 0};
                    ra[q] = (m0 + row < g.M) ? *reinterpret_cast<const v4i*>(Ai + (size_t)(m0 + row) * g.Kp + k0 + kc * 16) : zero;
                    rb[q] = (n0 + row < g.P) ? *reinterpret_cast<const v4i*>(Bj + (size_t)(n0 + row) * g.Kp + k0 + kc * 16) : zero;
                }
            };
            fetch(0);
            for (uint32_t k0 = 0; k0 < g.Kp; k0 += GBK) {
                __syncthreads();                    // every wave is done with the previous tile
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t c = t + 256 * q, row = c >> 3, kc = c & 7;
                    *reinterpret_cast<v4i*>(sA + row * GLD + kc * 16) = ra[q];
                    *reinterpret_cast<v4i*>(sB + row * GLD + kc * 16) = rb[q];
                }
                __syncthreads();
                if (k0 + GBK < g.Kp) fetch(k0 + GBK);
#pragma unroll
                for (int ks = 0; ks < GBK / 32; ++ks) {
                    const uint32_t ko = ks * 32 + 16 * (lane >> 5);
                    const v4i a0 = *reinterpret_cast<const v4i*>(sA + (wm * 64 + (lane & 31)) * GLD + ko);
                    const v4i a1 = *reinterpret_cast<const v4i*>(sA + (wm * 64 + 32 + (lane & 31)) * GLD + ko);
                    const v4i b0 = *reinterpret_cast<const v4i*>(sB + (wn * 64 + (lane & 31)) * GLD + ko);
                    const v4i b1 = *reinterpret_cast<const v4i*>(sB + (wn * 64 + 32 + (lane & 31)) * GLD + ko);
                    acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b1, acc[1], 0, 0, 0);
                    acc[2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b0, acc[2], 0, 0, 0);
                    acc[3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, acc[3], 0, 0, 0);
                }
            }
            const int shift = 8 * (i + j);
            if (shift < 64) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int r = 0; r < 16; ++r) tot[q][r] = (long long)((unsigned long long)tot[q][r] + ((unsigned long long)(long long)acc[q][r] << shift));
            }
        }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm * 64 + (q >> 1) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            const uint32_t col = n0 + wn * 64 + (q & 1) * 32 + (lane & 31);
            if (row < g.M && col < g.P) gemm_store(g, (b * g.M + row) * (size_t)g.P + col, tot[q][r]);
        }
}
// The same product for up to three planes a side (every projection and attention product of the LLaMa layer): all plane pairs
// are multiplied while a K tile lies in LDS, pairs of equal weight 256^(i+j) into one int32 accumulator (at most three pairs
// of at most K * 2^14 each; the caller keeps 3 K below 2^17), and the int64 recombination happens once, in the epilogue.
// Against the pair-by-pair kernel: one pass over the operands instead of PA * PB, PA * PB times the matrix instructions per
// barrier, no int64 totals held through the loop.  Block tile 64 x 64, one 32 x 32 tile per wave, two blocks per CU.
template <int PA, int PB> __global__ void __launch_bounds__(256, 2) k_gemm_i8_planes_all(const PlaneGemm g) {
    constexpr int NS = PA + PB - 1, TB = 64;
    __shared__ __attribute__((aligned(16))) int8_t sA[PA][TB * GLD];
    __shared__ __attribute__((aligned(16))) int8_t sB[PB][TB * GLD];
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
    const uint32_t m0 = blockIdx.y * TB, n0 = blockIdx.x * TB;
    const size_t b = blockIdx.z;
    const int8_t* __restrict__ A0 = g.A + (b * PA * g.M) * (size_t)g.Kp;
    const int8_t* __restrict__ B0 = g.B + (b * PB * g.P) * (size_t)g.Kp;
    const size_t a_plane = (size_t)g.M * g.Kp, b_plane = (size_t)g.P * g.Kp;
    v16i acc[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[s][r] = 0;
    v4i ra[PA][2], rb[PB][2];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t c = t + 256 * q, row = c >> 3, kc = c & 7;
            const v4i zero = {0, 0, 0, 0};
            const bool in_a = m0 + row < g.M, in_b = n0 + row < g.P;
            const size_t oa = (size_t)(m0 + row) * g.Kp + k0 + kc * 16, ob = (size_t)(n0 + row) * g.Kp + k0 + kc * 16;
#pragma unroll
            for (int i = 0; i < PA; ++i) ra[i][q] = in_a ? *reinterpret_cast<const v4i*>(A0 + i * a_plane + oa) : zero;
#pragma unroll
            for (int j = 0; j < PB; ++j) rb[j][q] = in_b ? *reinterpret_cast<const v4i*>(B0 + j * b_plane + ob) : zero;
        }
    };
    fetch(0);
    for (uint32_t k0 = 0; k0 < g.Kp; k0 += GBK) {
        __syncthreads();                    // every wave is done with the previous tile
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t c = t + 256 * q, row = c >> 3, kc = c & 7;
#pragma unroll
            for (int i = 0; i < PA; ++i) *reinterpret_cast<v4i*>(&sA[i][row * GLD + kc * 16]) = ra[i][q];
#pragma unroll
            for (int j = 0; j < PB; ++j) *reinterpret_cast<v4i*>(&sB[j][row * GLD + kc * 16]) = rb[j][q];
        }
        __syncthreads();
        if (k0 + GBK < g.Kp) fetch(k0 + GBK);
#pragma unroll
        for (int ks = 0; ks < GBK / 32; ++ks) {
            const uint32_t ko = ks * 32 + 16 * (lane >> 5);
            v4i fa[PA], fb[PB];
#pragma unroll
            for (int i = 0; i < PA; ++i) fa[i] = *reinterpret_cast<const v4i*>(&sA[i][(wm * 32 + (lane & 31)) * GLD + ko]);
#pragma unroll
            for (int j = 0; j < PB; ++j) fb[j] = *reinterpret_cast<const v4i*>(&sB[j][(wn * 32 + (lane & 31)) * GLD + ko]);
#pragma unroll
            for (int i = 0; i < PA; ++i)
#pragma unroll
                for (int j = 0; j < PB; ++j) acc[i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i + j], 0, 0, 0);
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        unsigned long long v = 0;
#pragma unroll
        for (int s = 0; s < NS; ++s) v += (unsigned long long)(long long)acc[s][r] << (8 * s);
        const uint32_t row = m0 + wm * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        const uint32_t col = n0 + wn * 32 + (lane & 31);
        if (row < g.M && col < g.P) gemm_store(g, (b * g.M + row) * (size_t)g.P + col, (long long)v);
    }
}
template <int PA> static bool launch_gemm_all_b(int pb, dim3 grid, hipStream_t st, const PlaneGemm& g) {
    switch (pb) {
        case 1: hipLaunchKernelGGL((k_gemm_i8_planes_all<PA, 1>), grid, dim3(256), 0, st, g); return true;
        case 2: hipLaunchKernelGGL((k_gemm_i8_planes_all<PA, 2>), grid, dim3(256), 0, st, g); return true;
        case 3: hipLaunchKernelGGL((k_gemm_i8_planes_all<PA, 3>), grid, dim3(256), 0, st, g); return true;
        default: return false;
    }
}
static bool launch_gemm_all(int pa, int pb, dim3 grid, hipStream_t st, const PlaneGemm& g) {
    switch (pa) {
        case 1: return launch_gemm_all_b<1>(pb, grid, st, g);
        case 2: return launch_gemm_all_b<2>(pb, grid, st, g);
        case 3: return launch_gemm_all_b<3>(pb, grid, st, g);
        default: return false;
    }
}
// Measurement: every launch of k_gemm_i8_planes between zk_prof_gemm_begin and zk_prof_gemm_read is timed with events on its stream.
struct GemmTimer { bool on = false; std::mutex mu; std::vector<std::pair<hipEvent_t, hipEvent_t>> ev; double macs = 0; };
static GemmTimer g_gemm_timer;
static const int g_gemm_timer_hook = (at_shutdown([] {
    std::lock_guard<std::mutex> lk(g_gemm_timer.mu);
    for (auto& e : g_gemm_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    g_gemm_timer.ev.clear();
    g_gemm_timer.on = false;
}), 0);
static int digits_for(unsigned long long absmax) {      // planes needed for |x| <= absmax: p digits reach 127 (256^p - 1) / 255
    int p = 1;
    unsigned __int128 reach = 127;
    while (reach < absmax && p < 8) { reach = reach * 256 + 127; ++p; }
    return reach >= absmax ? p : 0;
}
// returns ZK status; *done = false when the path does not apply (the caller then takes a VALU kernel)
// A right operand kept by the caller for many products (a layer's weight): its largest magnitude and, when it is a matrix of
// small integers, its digit planes in the GEMM's layout -- neither is computed again per product.
struct MatmulRhs { const void* B = nullptr; uint32_t N = 0, P = 0, Kp = 0; unsigned long long mb = ~0ull; int pb = 0; void* planes = nullptr; };
static int run_int8_plane_path(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, unsigned long long ma, unsigned long long mb,
                               hipStream_t st, bool* done, const MatmulRhs* rhs = nullptr, ProdSrc src = ProdSrc{nullptr, nullptr}, long long* C64 = nullptr,
                               bool b_transposed = false) {
    *done = false;
    const int pa = digits_for(ma), pb = digits_for(mb);
    if (!pa || !pb) return 0;
    if (N >= (1u << 17)) return 0;                                   // |sum_k of digit products| must stay below 2^31
    if (M > (1u << 30) || P > (1u << 30)) return 0;
    const uint32_t Kp = (N + GBK - 1) / GBK * GBK;
    const size_t rows_a = (size_t)batch * M;
    const bool have_b = rhs && rhs->planes && rhs->pb == pb && rhs->Kp == Kp && batch == 1;
    Scratch pla(rows_a * pa * Kp, st), plb(have_b ? 1 : (size_t)batch * pb * P * Kp, st);
    if (pla.rc) return pla.rc;
    if (plb.rc) return plb.rc;
    hipLaunchKernelGGL(k_split_rows, dim3(cdiv(rows_a * (Kp / 4), 256)), dim3(256), 0, st, pla.as<int8_t>(), (const Fr*)A, src, rows_a, M, N, Kp, pa);
    // a right operand given transposed ([batch][P][N]) has its planes' layout already: its rows are split like the left operand's
    if (!have_b && b_transposed)
        hipLaunchKernelGGL(k_split_rows, dim3(cdiv((size_t)batch * P * (Kp / 4), 256)), dim3(256), 0, st, plb.as<int8_t>(), (const Fr*)B, ProdSrc{nullptr, nullptr}, (size_t)batch * P, P, N, Kp, pb);
    else if (!have_b) hipLaunchKernelGGL(k_split_cols, dim3(cdiv(P, 64), Kp / 64, batch), dim3(256), 0, st, plb.as<int8_t>(), (const Fr*)B, N, P, Kp, pb);
    const PlaneGemm g{pla.as<int8_t>(), have_b ? (const int8_t*)rhs->planes : plb.as<int8_t>(), (Fr*)C, M, P, Kp, pa, pb, C64};
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (g_gemm_timer.on) {
        ZK_HIP(hipEventCreate(&t0));
        ZK_HIP(hipEventCreate(&t1));
        ZK_HIP(hipEventRecord(t0, st));
    }
    // up to three planes a side and three pairs' sums within int32: every pair in one pass; else pair by pair
    const bool all_pairs = pa <= 3 && pb <= 3 && 3ull * N < (1ull << 17) && launch_gemm_all(pa, pb, dim3(cdiv(P, 64), cdiv(M, 64), batch), st, g);
    if (!all_pairs) hipLaunchKernelGGL(k_gemm_i8_planes, dim3(cdiv(P, GBN), cdiv(M, GBM), batch), dim3(256), 0, st, g);
    if (g_gemm_timer.on) {
        ZK_HIP(hipEventRecord(t1, st));
        std::lock_guard<std::mutex> lk(g_gemm_timer.mu);
        g_gemm_timer.ev.emplace_back(t0, t1);
        g_gemm_timer.macs += (double)batch * M * N * P * pa * pb;
    }
    ZK_LAUNCH_CHECK();
    *done = true;
    return 0;
}
static inline unsigned absmax_grid(size_t n) {
    size_t b = n / (256 * 8) + 1;
    return (unsigned)(b > 1024 ? 1024 : b);
}

extern "C" {

int zk_fr_matmul_generic(void* C, const void* A, const void* B, uint32_t M, uint32_t N, uint32_t P, void* st) {
    if (M == 0 || P == 0) return 0;
    ZK_ARG(N > 0, "zk_fr_matmul: inner dimension is 0");
    hipLaunchKernelGGL(k_matmul, dim3(cdiv(P, TN), cdiv(M, TM)), dim3(TM * TN), 0, (hipStream_t)st, (Fr*)C, (const Fr*)A, (const Fr*)B, M, N, P);
    ZK_LAUNCH_CHECK();
    return 0;
}

// mode: 0 = choose (small-integer path when the device-side bound check allows it),
//       1 = always generic Montgomery, 2 = require the small-integer path (error if not applicable).
// path_used (optional, host): 1 generic, 2 small-integer.
// `batch` products of equally shaped matrices stored one after the other; the bound is taken over the whole stacks, so
// one path serves every product of the call
// src.a set: the left operand is the elementwise product of two int32 forms and A is null; the paths that need field elements
// get them written out first
static int matmul_dispatch(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used, void* stv,
                           const MatmulRhs* rhs = nullptr, ProdSrc src = ProdSrc{nullptr, nullptr}, long long* C64 = nullptr, bool b_transposed = false) {
    // C64 set: only the matrix-core path writes it; *path_used is 0 and nothing is written when that path does not apply
    hipStream_t st = (hipStream_t)stv;
    std::unique_ptr<Scratch> a_written;
    auto write_out = [&]() -> int {          // the product as field elements, once
        if (!src.a || A) return 0;
        a_written.reset(new Scratch(sizeof(Fr) * (size_t)batch * M * N, st));
        if (a_written->rc) return a_written->rc;
        const size_t na = (size_t)batch * M * N;
        hipLaunchKernelGGL(k_prod_to_fr, dim3(cdiv(na, 256)), dim3(256), 0, st, a_written->as<Fr>(), src, na);
        ZK_LAUNCH_CHECK();
        A = a_written->p;
        return 0;
    };
    if (batch == 0 || M == 0 || P == 0) return 0;
    ZK_ARG(N > 0, "zk_fr_matmul: inner dimension is 0");
    ZK_ARG((A != nullptr || src.a != nullptr) && B != nullptr && (C != nullptr || C64 != nullptr), "zk_fr_matmul: null operand or result");
    ZK_ARG(mode >= 0 && mode <= 2, "zk_fr_matmul: mode must be 0, 1 or 2");
    ZK_ARG(batch <= 65535, "zk_fr_matmul: at most 65535 products per call");
    ZK_ARG((size_t)batch * M < ((size_t)1 << 31), "zk_fr_matmul: too many rows in one call");
    bool small = false, fits32 = false, b_fits32 = false;
    unsigned long long ma_ = 0, mb_ = 0;
    if (mode != 1) {
        Scratch mx(3 * sizeof(unsigned long long), st);
        if (mx.rc) return mx.rc;
        ZK_HIP(hipMemsetAsync(mx.p, 0, 3 * sizeof(unsigned long long), st));
        const size_t nb = (size_t)batch * N * P;
        if (!rhs) hipLaunchKernelGGL(k_absmax, dim3(absmax_grid(nb)), dim3(256), 0, st, mx.as<unsigned long long>() + 1, (const Fr*)B, nb);
        if (src.a) hipLaunchKernelGGL(k_rowabs_prod, dim3(batch * M), dim3(256), 0, st, mx.as<unsigned long long>() + 2, mx.as<unsigned long long>(), src, N);
        else hipLaunchKernelGGL(k_rowabs, dim3(batch * M), dim3(256), 0, st, mx.as<unsigned long long>() + 2, mx.as<unsigned long long>(), (const Fr*)A, N);      // one pass over A for both of its figures
        ZK_LAUNCH_CHECK();
        void* stage = nullptr;
        int rc = staging(&stage, 24);
        if (rc) return rc;
        ZK_HIP(hipMemcpyAsync(stage, mx.p, 24, hipMemcpyDeviceToHost, st));
        ZK_HIP(hipStreamSynchronize(st));
        const unsigned long long ma = ((unsigned long long*)stage)[0], mb = rhs ? rhs->mb : ((unsigned long long*)stage)[1], ra = ((unsigned long long*)stage)[2];
        if (ma != ~0ull && mb != ~0ull && ra != ~0ull) {
            // |sum_j a_ij b_jk| <= (max_i sum_j |a_ij|) * max|b| must stay below 2^62
            const unsigned __int128 bound = (unsigned __int128)ra * mb;
            small = bound < ((unsigned __int128)1 << 62);
            fits32 = ma < (1ull << 31) && mb < (1ull << 31);
            b_fits32 = mb < (1ull << 31) && ma < (1ull << 62);
            ma_ = ma; mb_ = mb;
        }
        if (mode == 2 && !small) { set_error(ZK_ERR_ARG, "zk_fr_matmul: operands do not satisfy the small-integer bound"); return ZK_ERR_ARG; }
    }
    if (C64 && !small) { if (path_used) *path_used = 0; return 0; }
    if (mode == 1 || !small) { int wrc = write_out(); if (wrc) return wrc; }
    if (!small) {
        if (path_used) *path_used = 1;
        hipLaunchKernelGGL(k_matmul, dim3(cdiv(P, TN), cdiv(M, TM), batch), dim3(TM * TN), 0, st, (Fr*)C, (const Fr*)A, (const Fr*)B, M, N, P);
        ZK_LAUNCH_CHECK();
        return 0;
    }
    if (path_used) *path_used = 2;
    // large products go to the matrix cores as int8 digit planes; below ~1 G multiply-accumulates (over the whole stack)
    // the conversions outweigh the gain (ZKLLM_MATMUL_PLANES: log2 of that threshold, 0 = never)
    const char* planes_env = getenv("ZKLLM_MATMUL_PLANES");           // read at every call: tests lower it around single products
    const int planes_log2 = planes_env ? atoi(planes_env) : 30;
    if (planes_log2 > 0 && (unsigned __int128)batch * M * N * P >= ((unsigned __int128)1 << planes_log2) && M >= 32 && P >= 32) {
        bool done = false;
        const int rc = run_int8_plane_path(C, A, B, batch, M, N, P, ma_, mb_, st, &done, rhs, src, C64, b_transposed);
        if (rc) return rc;
        if (done) return 0;
    }
    if (C64) { if (path_used) *path_used = 0; return 0; }
    { int wrc = write_out(); if (wrc) return wrc; }
    if (fits32) return run_int_path<int>(C, A, B, batch, M, N, P, st);
    if (b_fits32) return run_wide_narrow_path(C, A, B, batch, M, N, P, st);
    return run_int_path<long long>(C, A, B, batch, M, N, P, st);
}
int zk_prof_gemm_begin(void) {
    std::lock_guard<std::mutex> lk(g_gemm_timer.mu);
    for (auto& e : g_gemm_timer.ev) { (void)hipEventDestroy(e.first); (void)hipEventDestroy(e.second); }
    g_gemm_timer.ev.clear();
    g_gemm_timer.macs = 0;
    g_gemm_timer.on = true;
    return 0;
}
// total_ms / launches: summed durations and number of the timed launches; macs: int8 multiply-accumulates they performed
// (rows x contraction x columns x plane pairs, without the padding)
int zk_prof_gemm_read(double* total_ms, unsigned long long* launches, double* macs) {
    std::lock_guard<std::mutex> lk(g_gemm_timer.mu);
    g_gemm_timer.on = false;
    double tot = 0;
    for (auto& e : g_gemm_timer.ev) {
        ZK_HIP(hipEventSynchronize(e.second));
        float ms = 0;
        ZK_HIP(hipEventElapsedTime(&ms, e.first, e.second));
        tot += ms;
    }
    *total_ms = tot;
    *launches = g_gemm_timer.ev.size();
    *macs = g_gemm_timer.macs;
    return 0;
}
// B (N x P) examined once for any number of products A * B: its largest magnitude, and its digit planes when it holds
// small integers.  B must stay alive and unmodified while the handle is in use.
int zk_fr_matmul_rhs_prepare(void** prepared, const void* B, uint32_t N, uint32_t P, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(prepared != nullptr && B != nullptr && N > 0 && P > 0, "zk_fr_matmul_rhs_prepare: null argument or empty matrix");
    std::unique_ptr<MatmulRhs> r(new MatmulRhs);
    r->B = B; r->N = N; r->P = P;
    r->Kp = (N + GBK - 1) / GBK * GBK;
    {
        Scratch mx(sizeof(unsigned long long), st);
        if (mx.rc) return mx.rc;
        ZK_HIP(hipMemsetAsync(mx.p, 0, sizeof(unsigned long long), st));
        const size_t nb = (size_t)N * P;
        hipLaunchKernelGGL(k_absmax, dim3(absmax_grid(nb)), dim3(256), 0, st, mx.as<unsigned long long>(), (const Fr*)B, nb);
        ZK_LAUNCH_CHECK();
        void* stage = nullptr;
        int rc = staging(&stage, 8);
        if (rc) return rc;
        ZK_HIP(hipMemcpyAsync(stage, mx.p, 8, hipMemcpyDeviceToHost, st));
        ZK_HIP(hipStreamSynchronize(st));
        r->mb = *(unsigned long long*)stage;
    }
    const int pb = r->mb == ~0ull ? 0 : digits_for(r->mb);
    if (pb && N < (1u << 17) && P <= (1u << 30)) {
        int rc = pool_alloc(&r->planes, (size_t)pb * P * r->Kp, st);
        if (rc) return rc;
        r->pb = pb;
        hipLaunchKernelGGL(k_split_cols, dim3(cdiv(P, 64), r->Kp / 64, 1), dim3(256), 0, st, (int8_t*)r->planes, (const Fr*)B, N, P, r->Kp, pb);
        if (hipGetLastError() != hipSuccess) { (void)pool_free(r->planes, st); return hip_fail(hipErrorLaunchFailure, "k_split_cols", __FILE__, __LINE__); }
    }
    *prepared = r.release();
    return 0;
}
int zk_fr_matmul_rhs_free(void* prepared) {
    MatmulRhs* r = (MatmulRhs*)prepared;
    if (!r) return 0;
    if (r->planes) (void)pool_free(r->planes, nullptr);
    delete r;
    return 0;
}
// zk_fr_matmul with a prepared right operand (its shape comes with the handle)
int zk_fr_matmul_rhs(void* C, const void* A, const void* prepared, uint32_t M, int mode, int* path_used, void* stv) {
    const MatmulRhs* r = (const MatmulRhs*)prepared;
    ZK_ARG(r != nullptr, "zk_fr_matmul_rhs: null handle");
    return matmul_dispatch(C, A, r->B, 1, M, r->N, r->P, mode, path_used, stv, r);
}
// the same with the left operand given by its int32 form (M * N int32 on the device): 4 bytes read per element instead of 32
int zk_fr_matmul_rhs_ints(void* C, const void* a_ints, const void* prepared, uint32_t M, int mode, int* path_used, void* stv) {
    const MatmulRhs* r = (const MatmulRhs*)prepared;
    ZK_ARG(r != nullptr && a_ints != nullptr, "zk_fr_matmul_rhs_ints: null argument");
    return matmul_dispatch(C, nullptr, r->B, 1, M, r->N, r->P, mode, path_used, stv, r, ProdSrc{(const int32_t*)a_ints, nullptr});
}
int zk_fr_matmul(void* C, const void* A, const void* B, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used, void* stv) {
    return matmul_dispatch(C, A, B, 1, M, N, P, mode, path_used, stv);
}
int zk_fr_matmul_batched(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used, void* stv) {
    return matmul_dispatch(C, A, B, batch, M, N, P, mode, path_used, stv);
}
// zk_fr_matmul_batched with the products written as 64-bit integers (C64: batch * M * P int64 on the device).  Only the
// matrix-core path does that: *taken_host is 1 when it ran, 0 when the operands or the shape do not allow it -- nothing is written then.
int zk_fr_matmul_batched_i64(void* C64, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int* taken_host, void* stv) {
    ZK_ARG(C64 != nullptr && taken_host != nullptr, "zk_fr_matmul_batched_i64: null argument");
    int path = 0;
    const int rc = matmul_dispatch(nullptr, A, B, batch, M, N, P, 0, &path, stv, nullptr, ProdSrc{nullptr, nullptr}, (long long*)C64);
    *taken_host = (rc == 0 && path == 2) ? 1 : 0;
    return rc;
}
// the same with the right operand given transposed (Bt: batch * P * N elements, Bt[b][p][k] = B[b][k][p]): Q K^T straight from K
int zk_fr_matmul_batched_i64_bt(void* C64, const void* A, const void* Bt, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int* taken_host, void* stv) {
    ZK_ARG(C64 != nullptr && taken_host != nullptr, "zk_fr_matmul_batched_i64_bt: null argument");
    int path = 0;
    const int rc = matmul_dispatch(nullptr, A, Bt, batch, M, N, P, 0, &path, stv, nullptr, ProdSrc{nullptr, nullptr}, (long long*)C64, true);
    *taken_host = (rc == 0 && path == 2) ? 1 : 0;
    return rc;
}
int zk_fr_matmul_batched_prod(void* C, const void* a_ints, const void* b_ints, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used, void* stv) {
    ZK_ARG(a_ints != nullptr && b_ints != nullptr, "zk_fr_matmul_batched_prod: null int32 form");
    return matmul_dispatch(C, nullptr, B, batch, M, N, P, mode, path_used, stv, nullptr, ProdSrc{(const int32_t*)a_ints, (const int32_t*)b_ints});
}

}  // extern "C"

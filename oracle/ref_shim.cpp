// TEST INFRASTRUCTURE ONLY.
//
// Builds the reference's own field/curve source (bls12-381.cu, its non-NVCC branch) as
// host C++ and exports a few C entry points so the restatement in ff.hpp can be checked
// bit-for-bit against the real thing.  The reference file is included where it lies
// (REF_BLS_SOURCE, an absolute path given by the Makefile); it is never copied.
// Output goes to oracle/_ref/ only.  This file cannot build where /root/reference is absent.
#include <sys/types.h>
#include <algorithm>
#include <cstdint>
typedef unsigned char uchar;
#define __kernel
#define __global
#define __local
#define __constant
static inline unsigned long mad_hi(unsigned long a, unsigned long b, unsigned long c) {
    return (unsigned long)(((unsigned __int128)a * b) >> 64) + c;
}
static inline uint get_global_id(int) { return 0; }
static inline uint get_group_id(int) { return 0; }
static inline uint get_local_id(int) { return 0; }
static inline uint get_local_size(int) { return 1; }
#define CLK_LOCAL_MEM_FENCE 0
static inline void barrier(int) {}
using std::max;
using std::min;
#include REF_BLS_SOURCE

typedef blstrs__scalar__Scalar RFr;
typedef blstrs__fp__Fp RFp;
typedef blstrs__g1__G1Affine_jacobian RJac;
typedef blstrs__g1__G1Affine_affine RAff;

extern "C" {
// op: 0 add, 1 sub, 2 mul (Montgomery product), 3 double(a), 4 mont(a), 5 unmont(a), 6 inverse(a) [mont in/out]
void ref_fr_op(int op, const RFr* a, const RFr* b, RFr* out, long n) {
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = blstrs__scalar__Scalar_add(a[i], b[i]); break;
        case 1: out[i] = blstrs__scalar__Scalar_sub(a[i], b[i]); break;
        case 2: out[i] = blstrs__scalar__Scalar_mul(a[i], b[i]); break;
        case 3: out[i] = blstrs__scalar__Scalar_double(a[i]); break;
        case 4: out[i] = blstrs__scalar__Scalar_mont(a[i]); break;
        case 5: out[i] = blstrs__scalar__Scalar_unmont(a[i]); break;
        case 6: out[i] = blstrs__scalar__Scalar_inverse(a[i]); break;
    }
}
void ref_fp_op(int op, const RFp* a, const RFp* b, RFp* out, long n) {
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = blstrs__fp__Fp_add(a[i], b[i]); break;
        case 1: out[i] = blstrs__fp__Fp_sub(a[i], b[i]); break;
        case 2: out[i] = blstrs__fp__Fp_mul(a[i], b[i]); break;
        case 3: out[i] = blstrs__fp__Fp_double(a[i]); break;
        case 4: out[i] = blstrs__fp__Fp_mont(a[i]); break;
        case 5: out[i] = blstrs__fp__Fp_unmont(a[i]); break;
    }
}
// op: 0 add(a,b), 1 double(a), 2 add_mixed(a, affine part of b)
void ref_g1_op(int op, const RJac* a, const RJac* b, RJac* out, long n) {
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = blstrs__g1__G1Affine_add(a[i], b[i]); break;
        case 1: out[i] = blstrs__g1__G1Affine_double(a[i]); break;
        case 2: { RAff q = {b[i].x, b[i].y}; out[i] = blstrs__g1__G1Affine_add_mixed(a[i], q); break; }
    }
}
void ref_constants(RFr* fr4, RFp* fp4, RFr* p_sub_2) {
    fr4[0] = blstrs__scalar__Scalar_ONE; fr4[1] = blstrs__scalar__Scalar_P;
    fr4[2] = blstrs__scalar__Scalar_R2;  fr4[3] = blstrs__scalar__Scalar_ZERO;
    fp4[0] = blstrs__fp__Fp_ONE; fp4[1] = blstrs__fp__Fp_P;
    fp4[2] = blstrs__fp__Fp_R2;  fp4[3] = blstrs__fp__Fp_ZERO;
    *p_sub_2 = blstrs__scalar__Scalar_P_sub_2;
}
// Single-thread multiply chain used when the reference build itself is the timed CPU baseline.
void ref_fr_mul_chain(const RFr* a, RFr* acc, long n) {
    RFr x = *acc;
    for (long i = 0; i < n; ++i) x = blstrs__scalar__Scalar_mul(x, a[i]);
    *acc = x;
}
}

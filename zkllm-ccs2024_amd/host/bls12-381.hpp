// Field / curve element types of the prover's host API.  Same names and memory layout as the
// reference's vendored types (bls12-381.cuh:116-120, :221-225, :424-433), so driver code written
// against Fr_t / G1Jacobian_t compiles unchanged.  The arithmetic itself lives in
// ../csrc/field.hpp (shared by the GPU kernels and the host-side scalar operators).
#pragma once
#include <cstdint>
#include <sys/types.h>

typedef unsigned int uint;

typedef struct { uint val[8]; } blstrs__scalar__Scalar;
typedef struct { uint val[12]; } blstrs__fp__Fp;
typedef struct { blstrs__fp__Fp x; blstrs__fp__Fp y; } blstrs__g1__G1Affine_affine;
typedef struct { blstrs__fp__Fp x; blstrs__fp__Fp y; blstrs__fp__Fp z; } blstrs__g1__G1Affine_jacobian;

typedef blstrs__scalar__Scalar Fr_t;
typedef blstrs__fp__Fp Fp_t;
typedef blstrs__g1__G1Affine_affine G1Affine_t;
typedef blstrs__g1__G1Affine_jacobian G1Jacobian_t;

static_assert(sizeof(Fr_t) == 32 && sizeof(G1Affine_t) == 96 && sizeof(G1Jacobian_t) == 144, "layout contract");

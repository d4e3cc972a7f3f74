/* zkllm_hip.h -- C ABI of the MI355X (gfx950) prover kernels.
 *
 * This is the boundary a host program binds to (the C++ class layer in
 * zkllm-ccs2024_amd/host does; so do the ctypes tests).  Plain pointers and sizes only.
 *
 * Conventions
 *   - Every function returns 0 on success, a hipError_t value or a code >= 10001 otherwise;
 *     zk_last_error() returns the message of the calling thread's last failure.  Nothing throws.
 *   - Pointers named out/a/b/in/table/... are DEVICE pointers unless the name ends in _host
 *     or the parameter is a `const uint32_t*` scalar/challenge (8 limbs per Fr, host memory).
 *   - Fr element: 8 little-endian u32 limbs, 32 bytes, standard (non-Montgomery) form -- the
 *     reference's Fr_t as stored by FrTensor (fr-tensor.cuh:15, fr-tensor.cu:181-184).
 *   - G1 point: Jacobian (x,y,z), 3 x 12 u32 limbs, Montgomery form, 144 bytes -- the reference's
 *     G1Jacobian_t as stored by G1TensorJacobian (bls12-381.cuh:429-433, g1-tensor.cu:174-183).
 *     Any z == 0 is the point at infinity.
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream).  Launches are
 *     asynchronous; functions that return host values synchronise that stream.
 *   - Scratch memory comes from the library's caching allocator (zk_malloc/zk_free).  The allocator
 *     remembers for every freed block the stream of its last user and makes a new user on another
 *     stream wait for it, so entry points may be called on different streams.  zk_free assumes the
 *     default stream; name another with zk_free_async.  Host threads may call concurrently (errors
 *     and staging buffers are per thread); a *_begin / *_end pair belongs to one thread.
 */
#ifndef ZKLLM_HIP_H
#define ZKLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- runtime ------------------------------------------------------------------------------- */
const char* zk_last_error(void);
int zk_init(int device);                                   /* hipSetDevice; fails if no GPU */
int zk_device_info(char* name, int name_len, int* compute_units, int* clock_khz, size_t* total_mem);
/* replaces the cudaMalloc/cudaFree pair of every FrTensor/G1Tensor ctor/dtor (fr-tensor.cu:158-179) */
int zk_malloc(void** out, size_t bytes);
int zk_free(void* p);                                      /* last user: the default stream */
int zk_free_async(void* p, void* stream);                  /* last user: kernels already queued on `stream` */
int zk_pool_trim(void);                                    /* return cached blocks to the driver */
int zk_pool_stats(size_t* live_bytes, size_t* cached_bytes);
/* No counterpart in the reference (which leaves everything to process exit): waits for the device and releases, in a fixed
 * order and while the runtime is alive, what the library itself holds -- timing events, the cached eq table, cached blocks
 * (live blocks stay with their owners), its streams, the allocator's events, idle pinned buffers.  The library stays usable
 * afterwards.  A host calls it before it exits so that nothing is left to static destruction. */
int zk_shutdown(void);
/* No counterpart in the reference.  The sumcheck jobs that run beside the caller (zk_lookup_prove_begin*, zk_hadamard_prove_begin*)
 * are long sequences of launches on a stream of the library's own.  With this on (the default; ZKLLM_ASYNC_JOBS=0 in the
 * environment turns it off) begin only orders the job behind the caller's stream and hands the launches to a thread of the
 * library's, so the caller goes on queuing its own work at once; the matching end waits for that thread to be done with the
 * job before it waits for the device.  Results are the same either way.  An error met while the job's launches are queued is
 * reported by its end call.  Jobs are launched in the order of their begin calls. */
int zk_set_async_jobs(int on);
int zk_async_jobs(void);
/* No counterpart in the reference.  Deferred results: between zk_defer_begin and zk_defer_end (same host thread), the entry points
 * that hand a few field elements back to the host -- zk_fr_me, zk_fr_me_multi(_ints), zk_ip_round, zk_ip_sumcheck_small -- queue
 * their kernels and the copy of their results and return WITHOUT waiting and WITHOUT writing their host output arguments;
 * zk_defer_end records an event on `stream` (the stream those calls were given) and zk_defer_wait waits for it and writes every
 * result, in the order of the calls and with each call's own layout, to out_host (n_fr: how many field elements; at most 2048
 * per batch).  For a caller that knows all its challenges and wants a chain of such calls queued in one go, e.g. the device
 * side of a whole zkFC proof (zkfc.cu:61-87), and collects the values where the transcript needs them.  Other entry points are
 * not affected.  zk_defer_free releases the batch (waiting for its copies first); one open batch per thread. */
int zk_defer_begin(void** batch);
int zk_defer_end(void* batch, void* stream);
int zk_defer_wait(void* batch, uint32_t* out_host, size_t max_fr, size_t* n_fr);
int zk_defer_free(void* batch);
/* replace cudaMemcpy in ctors, operator()(idx), savebin/loadbin (ioutils.cu:3-45) */
int zk_memcpy_h2d(void* dst, const void* src_host, size_t bytes, void* stream);
int zk_memcpy_d2h(void* dst_host, const void* src, size_t bytes, void* stream);
int zk_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int zk_memset(void* dst, int value, size_t bytes, void* stream);
int zk_sync(void* stream);
int zk_event_create(void** ev);
int zk_event_destroy(void* ev);
int zk_event_record(void* ev, void* stream);
int zk_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- Fr elementwise (Fr_elementwise_* / Fr_broadcast_*, fr-tensor.cu:71-153, :257-373) ------- */
int zk_fr_add(void* out, const void* a, const void* b, size_t n, void* stream);
int zk_fr_sub(void* out, const void* a, const void* b, size_t n, void* stream);
int zk_fr_mul(void* out, const void* a, const void* b, size_t n, void* stream);       /* a*b (Fr_elementwise_mul) */
int zk_fr_montmul(void* out, const void* a, const void* b, size_t n, void* stream);   /* a*b*R^-1 (Fr_elementwise_mont_mul) */
int zk_fr_neg(void* out, const void* a, size_t n, void* stream);
int zk_fr_add_s(void* out, const void* a, const uint32_t* s, size_t n, void* stream);
int zk_fr_sub_s(void* out, const void* a, const uint32_t* s, size_t n, void* stream);
int zk_fr_mul_s(void* out, const void* a, const uint32_t* s, size_t n, void* stream);
int zk_fr_mont(void* out, const void* a, size_t n, void* stream);                     /* a*R  */
int zk_fr_unmont(void* out, const void* a, size_t n, void* stream);                   /* a/R  */
int zk_fr_fill(void* out, const uint32_t* s, size_t n, void* stream);
int zk_fr_bias_add(void* z, const void* bias, size_t rows, uint32_t cols, void* stream);   /* fcAddBiasKernel zkfc.cu:36-41 */

/* ---- conversions (fr-tensor.cu:186-248, :691-798, :922-945) ------------------------------------ */
int zk_fr_from_i32(void* out, const void* in_i32, size_t n, void* stream);
int zk_fr_from_i64(void* out, const void* in_i64, size_t n, void* stream);
int zk_fr_from_u32(void* out, const void* in_u32, size_t n, void* stream);             /* count_to_m tlookup.cu:17-20 */
int zk_fr_from_f32(void* out, const void* in_f32, uint64_t scaling_factor, size_t n, void* stream);
int zk_fr_from_f64(void* out, const void* in_f64, uint64_t scaling_factor, size_t n, void* stream);
int zk_fr_to_i32(void* out_i32, const void* in, size_t n, void* stream);
int zk_fr_to_i64(void* out_i64, const void* in, size_t n, void* stream);
/* out_f64[r] = sum_j (X[r][j] / scale)^2 in double precision, terms added in index order (the mean square that
 * llama-rmsnorm.py:38-39 computes with torch before calling the prover).  out_f64: rows doubles on the device. */
int zk_row_sumsq_f64(void* out_f64, const void* X, uint32_t rows, uint32_t cols, double scale, void* stream);

/* ---- layout (pad fr-tensor.cu:800-828, transpose :885-900, gather tlookup.cu:446-453) ----------- */
int zk_fr_pad(void* out, const void* in, size_t rows, uint32_t last_in, uint32_t last_out, const uint32_t* pad, void* stream);
int zk_fr_transpose(void* out, const void* in, uint32_t M, uint32_t N, void* stream);
/* the same for a stack of `batch` M x N matrices stored one after the other (per-head K^T of zkAttn::compute, zksoftmax.cu:234) */
int zk_fr_transpose_batched(void* out, const void* in, uint32_t batch, uint32_t M, uint32_t N, void* stream);
/* out[b][a][c] = in[a][b][c] (A x B x C elements): what self-attn.cu:80-90 reaches per head through transposes and slices, for
 * all heads at once -- [token][head][k] to [head][token][k] and back -- in one pass instead of two transposes */
int zk_fr_swap_axes(void* out, const void* in, uint32_t A, uint32_t B, uint32_t C, void* stream);
int zk_fr_gather(void* out, const void* table, const void* idx_u32, size_t n, void* stream);
/* dst[i] = src[offset + i * stride], i < count, for elements of elem_bytes (a multiple of 16: field elements, G1 points):
 * every 2^k-th column of a row-major tensor or generator vector (no counterpart in the reference; the cross commitments
 * of zk_g1_open_begin_batch_rows are commitments of such parts). */
int zk_copy_strided(void* dst, const void* src, size_t elem_bytes, size_t count, size_t stride, size_t offset, void* stream);

/* ---- reductions and folds ------------------------------------------------------------------------ */
/* FrTensor::sum (fr-tensor.cu:382-434) */
int zk_fr_sum(uint32_t* out_host, const void* a, size_t n, void* stream);
/* zk_fr_sum for callers that cannot allocate.  No counterpart in the reference: it is for code under HIP stream capture,
 * tight serving loops and harnesses that forbid hipMalloc.  Calls no hipMalloc/hipFree or any other allocating routine
 * and does not synchronise: the block partials that zk_fr_sum keeps in a pool block live in a 64 KiB device array inside
 * the library (one per GPU, held until the process ends), and the sum is written to out_dev, ONE Fr element on the
 * device (standard form), behind the work already queued on `stream`.  n <= ZK_FR_SUM_STATIC_MAX_N, else an error.
 * Every call on a GPU uses that GPU's one array: calls that overlap on the same GPU (two streams or two host threads)
 * race.  zk_init looks the array's address up for its device; otherwise the first call on a device does. */
#define ZK_FR_SUM_STATIC_MAX_N ((size_t)0xFFFFFFFFu)       /* the reference's tensor sizes are `uint` */
int zk_fr_sum_static(void* out_dev, const void* a, size_t n, void* stream);
/* sum_i a_i*b_i; replaces (a*b).sum() at tlookup.cu:360 */
int zk_fr_dot(uint32_t* out_host, const void* a, const void* b, size_t n, void* stream);
/* 1..3 levels of Fr_multi_dim_partial_me_step / Fr_me_step / Fr_partial_me_step in one pass over
 * in[other][cur][window] (fr-tensor.cu:518-560, :588-641).  u: `levels` standard-form challenges. */
int zk_fr_fold_axis(void* out, const void* in, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* stream);
/* A tensor that is folded again and again at new points and never changes (a layer's weight: the multilinear evaluations
 * of zkFC::prove, zkfc.cu:77-78, and the fold over the committed rows at the head of Commitment::me_open, commitment.cu:
 * 118-123), examined once: when every element is a 32-bit signed integer (fixed-point weights are) the handle keeps the int32
 * form, an eighth of the bytes, and *prepared is non-null; otherwise *prepared is left null (not an error) and the caller
 * folds the tensor itself.  No counterpart in the reference, which re-reads the field elements each time.  Synchronises.
 * zk_fr_fold_axis_prepared is all `levels` (1..24) levels of zk_fr_fold_axis at once for such a tensor read as
 * in[other][cur][window] with cur <= 2^levels (elements beyond cur count as zero):
 * out[o][w] = sum_j eq(u, j) in[o][j][w], u[0] on the lowest bit of j; bit-identical to the level-by-level fold. */
int zk_fr_fold_prepare(void** prepared, const void* t, size_t n, void* stream);
int zk_fr_fold_axis_prepared(void* out, const void* prepared, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* stream);
/* the same fold of the elementwise product of two such tensors (handles of equal size): out[o][w] = sum_j eq(u, j) a[o][j][w] b[o][j][w] */
int zk_fr_fold_axis_prod(void* out, const void* a_prepared, const void* b_prepared, const uint32_t* u, int levels, size_t other, uint32_t cur, size_t window, void* stream);
int zk_fr_fold_prepared_free(void* prepared);
/* The same handle for a tensor whose int32 form is written by the kernel that makes the tensor (the digit planes of
 * zk_softmax_decompose_ints, the outputs of zk_fr_gather_ints), so no pass over the field elements is needed: _new
 * allocates the handle and its n int32 slots (uninitialised) and returns their device address; the caller must have queued
 * the kernel that sets ints_dev[i] to element i before the handle is used.  _ints returns that address (null for null).
 * The int32 form must not change once that kernel has written it: other handles may remember what they were gathered from by
 * this one's identity (zk_fr_gather_by_queries_ints).  A caller that does write ints_dev again calls _touch afterwards: the handle
 * then counts as a new form and nothing gathered from the old one is trusted any more.  No counterpart in the reference. */
int zk_fr_fold_prepared_new(void** prepared, void** ints_dev, size_t n, void* stream);
const void* zk_fr_fold_prepared_ints(const void* prepared);
int zk_fr_fold_prepared_touch(void* prepared);
/* zk_fr_gather (out[i] = table[idx[i]], the mapped values of tLookupRangeMapping::operator(), tlookup.cu:446-470) that
 * also writes the int32 form of out from the table's own (table_prepared: a handle of zk_fr_fold_prepare over the table) */
int zk_fr_gather_ints(void* out, void* out_ints, const void* table, const void* table_prepared, const void* idx, size_t n, void* stream);
/* the same gather by the queries themselves: out[i] = table[queries[i] - low], queries and table given by their int32 forms,
 * out_prepared a handle of zk_fr_fold_prepared_new that receives out's int32 form (a query outside the table reads entry 0:
 * zk_lookup_index_i32, run before, reports those).  The handle remembers what it was gathered from: a mapped lookup job over
 * these queries, these outputs and this table (zk_lookup_prove_begin_mapped_ints) then knows that every output is its
 * query's table value and reads neither the outputs nor the per-entry integers in its first round.  out may be null: only the
 * int32 form is written then (for outputs whose readers all take that form). */
int zk_fr_gather_by_queries_ints(void* out, void* out_prepared, const void* queries_prepared, int32_t low, const void* table_prepared, size_t n, void* stream);
/* zk_fr_me_multi where prepareds[i], when non-null, is the int32 form of Xs[i] (same n): such tensors are read from it --
 * an eighth of the bytes, eight limb products per element instead of a Montgomery product.  Same values. */
/* zk_fr_mul (out = a * b element by element) for two tensors given by their int32 forms: the products are exact 64-bit
 * integers, no field multiplication and an eighth of the bytes read */
int zk_fr_mul_ints(void* out, const void* a_prepared, const void* b_prepared, size_t n, void* stream);
int zk_fr_me_multi_ints(uint32_t* out_host, const void* const* Xs, const void* const* prepareds, int K, size_t n, const uint32_t* u, int k, void* stream);
/* FrTensor::operator()(u) / Fr_me (fr-tensor.cu:437-442, :602-609): whole evaluation, fused */
int zk_fr_me(uint32_t* out_host, const void* a, size_t n, const uint32_t* u, int k, void* stream);
/* zkip_reduce_kernel / tLookup reduce kernels / hadamard_reduce_kernel on one tensor */
int zk_fr_fold_halves(void* out, const void* a, const uint32_t* v, size_t n_in, size_t n_out, void* stream);

/* ---- matmul (matrixMultiplyOptimized fr-tensor.cu:831-881) ---------------------------------------- */
int zk_fr_matmul_generic(void* C, const void* A, const void* B, uint32_t M, uint32_t N, uint32_t P, void* stream);
/* mode 0: pick the small-integer path when a device-side bound check proves it exact; 1: generic
 * Montgomery only; 2: small-integer only (error if the bound fails).  path_used: 1 generic, 2 small-int. */
int zk_fr_matmul(void* C, const void* A, const void* B, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used_host, void* stream);
/* the same for a stack of `batch` products, A [batch][M][N], B [batch][N][P], C [batch][M][P] (the per-head products of
 * zkAttn::compute, zksoftmax.cu:234-238, for all heads at once); the bound check covers the whole stacks, so one path serves all */
int zk_fr_matmul_batched(void* C, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used_host, void* stream);
/* the same for a left operand that is the elementwise product of two tensors given by their int32 forms (device pointers
 * to batch * M * N int32 each, zk_fr_fold_prepared_ints): the product, an exact 64-bit integer per element, is read where A
 * would be and written out as field elements only for the paths that read nothing else.  No counterpart in the reference
 * (zkSoftmax::compute multiplies the segments' table values into a tensor first, zksoftmax.cu:160-166). */
int zk_fr_matmul_batched_prod(void* C, const void* a_ints, const void* b_ints, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int mode, int* path_used_host,
                              void* stream);
/* zk_fr_matmul_batched with the products written as 64-bit integers (C64: batch * M * P int64 on the device), for a product whose
 * only reader takes that form (the attention scores, read once by zk_softmax_shift_decompose_i64).  Only the matrix-core path does
 * that: *taken_host is 1 when it ran, 0 when the operands or the shape do not allow it -- nothing is written then and the caller
 * falls back to zk_fr_matmul_batched.  No counterpart in the reference (zkAttn::compute, zksoftmax.cu:237-243, writes field elements). */
int zk_fr_matmul_batched_i64(void* C64, const void* A, const void* B, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int* taken_host, void* stream);
/* the same with the right operand given transposed (Bt[b][p][k] = B[b][k][p], batch * P * N elements): Q K^T straight from K */
int zk_fr_matmul_batched_i64_bt(void* C64, const void* A, const void* Bt, uint32_t batch, uint32_t M, uint32_t N, uint32_t P, int* taken_host, void* stream);
/* The right operand of many products (a layer's weight in zkFC::operator(), zkfc.cu:44-58) examined once: its largest magnitude
 * for the small-integer bound and, when it holds small integers, its int8 digit planes in the GEMM's layout.  No counterpart in
 * the reference, which converts nothing.  B stays alive and unmodified while the handle is used; zk_fr_matmul_rhs is
 * zk_fr_matmul(C, A, B, M, N, P, ...) with B's part of the preparation taken from the handle (bit-identical results). */
int zk_fr_matmul_rhs_prepare(void** prepared, const void* B, uint32_t N, uint32_t P, void* stream);
int zk_fr_matmul_rhs(void* C, const void* A, const void* prepared, uint32_t M, int mode, int* path_used, void* stream);
/* the same for a left operand given by its int32 form (M * N int32 on the device, zk_fr_fold_prepared_ints): the bound pass and the
 * digit planes read 4 bytes per element; the paths that read field elements get them written out first.  Same C. */
int zk_fr_matmul_rhs_ints(void* C, const void* a_ints, const void* prepared, uint32_t M, int mode, int* path_used_host, void* stream);
int zk_fr_matmul_rhs_free(void* prepared);

/* ---- inner-product sumcheck (zkip_poly_kernel + 3 sums, zkfc.cu:94-138) ----------------------------- */
int zk_ip_round(uint32_t* poly3_host, const void* a, const void* b, size_t n_in, size_t n_out, void* stream);
/* zkip_stacked_step_poly (zkfc.cu:187-209): halves over the stacking axis of [N][D] tensors, rows weighted by the eq table E */
int zk_ip_round_stacked(uint32_t* poly3_host, const void* a, const void* b, const void* E, size_t D, size_t rows_in, size_t rows_out, void* stream);
/* all rounds of zkip (zkfc.cu:140-151) in one launch, n <= 8192 */
int zk_ip_sumcheck_small(uint32_t* polys_host, uint32_t* fin_host, const void* a, const void* b, uint32_t n, const uint32_t* u, int k, void* stream);

/* ---- G1 tensors (g1-tensor.cu) ------------------------------------------------------------------------ */
int zk_g1_fill(void* out, const uint32_t* point36, size_t n, void* stream);               /* G1Jacobian_assign_broadcast :140 */
int zk_g1_neg(void* out, const void* a, size_t n, void* stream);                          /* G1_jacobian_elementwise_minus :192 */
int zk_g1_affine_neg(void* out, const void* a_affine, size_t n, void* stream);            /* G1_affine_elementwise_minus :105 */
int zk_g1_affine_to_jacobian(void* out, const void* a_affine, size_t n, void* stream);    /* G1_affine_to_jacobian :154 */
/* G1_jacobian_{elementwise,broadcast}_{add,sub} :207-320; b_count = n or 1 (b is a device pointer either way) */
int zk_g1_add(void* out, const void* a, const void* b, size_t n, size_t b_count, int subtract, void* stream);
/* G1_jacobian_{elementwise,broadcast}_{madd,msub}: b in affine form (96 B per point) */
int zk_g1_madd(void* out, const void* a, const void* b_affine, size_t n, size_t b_count, int subtract, void* stream);
/* out[i] = [s[i]] g[i % ng], s = Fr tensor read as 256-bit integers (G1_jacobian_elementwise_mul[_broadcast] :456-482) */
int zk_g1_scalar_mul(void* out, const void* g, const void* s_fr, size_t ng, size_t n, void* stream);
/* out[i] = [s_i] B for ONE base point B (host pointer: 36 limbs, Jacobian, Montgomery form) and n scalars in standard
 * form on the device: the broadcast G1Jacobian_mul of Commitment::random (commitment.cu:3-8, the generator times random
 * scalars; g1-tensor.cu:469-482).  Fixed-base windows: 33 mixed additions per scalar out of a table of B's multiples that
 * stays on the device between calls with the same base.  Results equal zk_g1_scalar_mul's as group elements. */
int zk_g1_fixed_base_mul(void* out, const uint32_t* base_host, const void* s_fr, size_t n, void* stream);
int zk_g1_sum(uint32_t* out_host36, const void* a, size_t n, void* stream);               /* G1TensorJacobian::sum :391-443 */
int zk_g1_rowwise_sum(void* out, const void* in, size_t nrow, size_t ncol, void* stream); /* rowwise_sum :535-625 */
int zk_g1_me(uint32_t* out_host36, const void* a, size_t n, const uint32_t* u, int k, void* stream);   /* G1_me :486-514 */
/* (x/z^2, y/z^3, ONE); infinity -> all-zero limbs.  Not in the reference (it has no Fp inversion);
 * used to compare and store points in a byte-stable form. */
int zk_g1_normalize(void* out, const void* in, size_t n, void* stream);

/* ---- Pedersen commitment (commitment.cu) ------------------------------------------------------------------ */
/* Commitment::commit_int :31-58 -- out[row] = sum_j [t[row*ngen + j]] gens[j]; t holds embedded int32 values */
int zk_g1_commit_int(void* out, const void* gens, const void* scalars_fr, size_t m, size_t ngen, void* stream);
/* one round of Commitment::me_open (me_open_step :79-107 + the three G1 sums :125-127) */
int zk_g1_open_round(void* new_scalars, void* new_gens, uint32_t* sums_host108, const void* scalars, const void* gens, const uint32_t* u, size_t old_size, void* stream);
/* the whole recursion of Commitment::me_open :109-129: `rounds` halvings of (scalars, gens) of length n with the
 * challenges u[0..rounds) (8 limbs each, host).  proof_host: 3*rounds+1 points of 36 limbs -- T, T0, T1 per round,
 * then the folded generator -- normalised to z = 1; final_scalar_host: the folded scalar (8 limbs).  The generators
 * must lie in the order-r subgroup (Commitment::random, :9-20, only produces such points). */
int zk_g1_open(uint32_t* proof_host, uint32_t* final_scalar_host, const void* scalars, const void* gens, size_t n, const uint32_t* u, int rounds, void* stream);
/* zk_g1_open in two halves, for callers that prove on while a weight is being opened (the reference opens each weight
 * in place, verifyWeightClaim proof.cu:9-15; the opening depends on nothing the prover does afterwards).  begin
 * queues the recursion on a stream of the library's own, ordered after the work queued on `stream` so far, and
 * returns; scalars and gens must stay alive and unmodified until end.  end waits, delivers what zk_g1_open
 * delivers, and releases the opening's buffers; every handle must be ended exactly once. */
int zk_g1_open_begin(void** handle, const void* scalars, const void* gens, size_t n, const uint32_t* u, int rounds, void* stream);
int zk_g1_open_end(void* handle, uint32_t* proof_host, uint32_t* final_scalar_host);
/* The generators of me_open (commitment.cu:109-129 takes the Commitment itself) in the form the rounds work on, made once
 * for any number of openings against them: affine points in 29-bit limbs and the first round's pair sums (1.5 n points
 * of 112 bytes; nothing in it depends on the opened tensor) and, above 1024 generators, the fixed-base tables of the
 * first two rounds' folds (255 points per generator pair for the first round, as much again for the second when it
 * folds more than 1024 generators: 28 KB per generator in all, kept until the handle is freed; building them takes
 * about as much again in temporaries).  zk_g1_open_begin_prepared is zk_g1_open_begin with
 * such generators; the handle must outlive every opening started with it and is released with
 * zk_g1_open_prepared_free. */
int zk_g1_open_prepare(void** prepared, const void* gens, size_t n, void* stream);
/* zk_g1_open_prepare with the choice of tables: 0 none, 1 / 2 those of the first / first two fold rounds (2 is what
 * zk_g1_open_prepare makes), 3 the tables of a fold that takes three rounds at once (seven differences per eight
 * generators; as large as the other two together, made in their place).  The three-round fold serves openings started with
 * zk_g1_open_begin_batch_rows and cross_rounds >= 3, whose first three rounds read no folded generators; any other opening
 * over such a handle folds by the walk.  Needs a power of two of at least 16384 generators, else 3 means 2. */
int zk_g1_open_prepare_tables(void** prepared, const void* gens, size_t n, int tables, void* stream);
/* The same with a byte budget for the tables instead of a fixed choice (no counterpart in the reference): makes the richest
 * mode <= want whose tables fit max_table_bytes (3: 24990 B per generator, 2: 28560, 1: 14280, 0: none) and reports it in
 * *tables_made (may be null).  _table_bytes: what a mode would keep for n generators; _prepared_table_bytes: what a handle keeps. */
int zk_g1_open_prepare_budget(void** prepared, const void* gens, size_t n, int want, size_t max_table_bytes, int* tables_made, void* stream);
size_t zk_g1_open_table_bytes(size_t n, int tables);
size_t zk_g1_open_prepared_table_bytes(const void* prepared);
int zk_g1_open_prepared_free(void* prepared);
int zk_g1_open_begin_prepared(void** handle, const void* scalars, const void* prepared, const uint32_t* u, int rounds, void* stream);
/* `count` (1..8) openings against prepared generator sets of ONE size with ONE round count as a single job: every kernel
 * of a halving round is launched once for all of them (the reference opens weight after weight, proof.cu:9-15; openings
 * are independent of each other).  scalars[i] / prepared[i]: opening i; u: its challenges at u + i * rounds * 8.  end
 * delivers opening i's points at proof_host + i * (3 rounds + 1) * 36 and its folded scalar at final_scalar_host + i * 8. */
int zk_g1_open_begin_batch(void** handle, int count, const void* const* scalars, const void* const* prepared, const uint32_t* u, int rounds, void* stream);
/* zk_g1_open_begin_batch for openings as Commitment::open makes them (commitment.cu:133-141): the opened vector is the
 * tensor's rows folded at u_out, and the reference evaluates the row commitments there too (com(u_out), :137).
 * rows[i]: commitments of tensor i's nrows[i] rows (Jacobian, 36 limbs each, on the device, alive until end), laid out
 * [pattern][row]: pattern 0 the row commitments C_r = sum_i W[r][i] g_i; with cross_rounds = R > 0 they are followed, for
 * q = 0 .. R-1, by the 4^q patterns p = a 2^q + b of T0_q, X[r] = sum_j W[r][2^(q+1) j + a] g_(2^(q+1) j + 2^q + b), and the
 * 4^q of T1_q, X[r] = sum_j W[r][2^(q+1) j + 2^q + a] g_(2^(q+1) j + b): 1 + 2 (4^R - 1) / 3 patterns in all (the host
 * layer's Commitment::cross_commitments makes them with commit_int over strided parts).  u_rows[i]: the k_rows[i] challenges
 * the rows were folded with, lowest row bit first, 2^k_rows >= nrows.
 * T of the first round is then sum_r eq(u_rows, r) C_r, and T0, T1 of the first R halving rounds are the combinations
 * of the cross patterns with the products of the earlier rounds' challenges -- sums over rows x patterns points instead
 * of bucket sums over all generators; those rounds then consist of their fold alone.  The points equal the sums over the
 * generators whenever rows[i] are such commitments of the tensor under these generators -- the caller's statement;
 * with other points T, T0, T1 of the halving rounds differ from zk_g1_open_begin_batch's, nothing else does. */
int zk_g1_open_begin_batch_rows(void** handle, int count, const void* const* scalars, const void* const* prepared, const uint32_t* u, int rounds,
                                const void* const* rows, const uint32_t* nrows, const uint32_t* const* u_rows, const int* k_rows, int cross_rounds, void* stream);
int zk_g1_open_end_batch(void* handle, uint32_t* proof_host, uint32_t* final_scalar_host);

/* ---- lookup argument (tlookup.cu) ------------------------------------------------------------------------ */
/* idx = val - low as a table index (lookuprange_tensor_prep_kernel :414-421 / lookuprange_prep_kernel :393-400);
 * unlike the reference, a value outside [low, low+table_size) is an error instead of an unchecked access */
int zk_lookup_index_fr(void* idx_u32, const void* vals_fr, int32_t low, uint32_t table_size, size_t n, void* stream);
int zk_lookup_index_i32(void* idx_u32, const void* vals_i32, int32_t low, uint32_t table_size, size_t n, void* stream);
/* multiplicities (tlookup_kernel :10-15): counts[b] = #{i : idx[i] == b}; counts is cleared first */
int zk_lookup_hist(void* counts_u32, const void* idx_u32, size_t n, uint32_t nbins, void* stream);
/* zk_lookup_index_i32 and zk_lookup_hist in one (tLookupRange::prep over queries that keep an int32 form): the counting passes
 * form the positions value - low themselves and no array of positions is written; a value outside [low, low + len) is an error */
int zk_lookup_hist_i32(void* counts_u32, const void* vals_i32, int32_t low, uint32_t len, size_t n, uint32_t nbins, void* stream);
int zk_range_table(void* table_fr, int32_t low, uint32_t len, uint32_t table_size, void* stream);   /* tlookuprange_init_kernel :372-380 */
/* out[i] = 1/(in[i]+beta) (tlookup_inv_kernel :50-62), by batch inversion */
int zk_fr_batch_inv(void* out, const void* in, const uint32_t* beta, size_t n, void* stream);
/* eq(u, t) for t < 2^k in Montgomery form; zk_eq_halve drops the top variable */
int zk_eq_table(void* out, const uint32_t* u, int k, void* stream);
int zk_eq_halve(void* out, const void* in, size_t n_out, void* stream);
/* FrTensor::operator()(u) (Fr_me fr-tensor.cu:602-609) for up to 8 tensors of n elements at the same point in one pass:
 * out_host[i] = multilinear extension of Xs[i] at u (k challenges, 2^(k-1) < n <= 2^k) */
int zk_fr_me_multi(uint32_t* out_host, const void* const* Xs, int K, size_t n, const uint32_t* u, int k, void* stream);
/* one sumcheck round: every sum of tLookup_phase1_step_poly :184-200 / tLookup_phase2_step_poly :245-279 plus the
 * folds of tLookup_phase1_reduce_kernel :94-103 / tLookup_phase2_reduce_kernel :161-175.
 * sums_host (standard form): [E.(a0 s0), E.(da s0 + a0 ds), E.(da ds), sum a0, sum da] and, in phase 2,
 * the same three for (B,T) followed by [sum m0 b0, sum (dm b0 + m0 db), sum dm db];  s0 = S + beta, E = eq table. */
int zk_lookup_round(uint32_t* sums_host, void* new_A, void* new_S, void* new_B, void* new_T, void* new_m,
                    const void* A, const void* S, const void* B, const void* T, const void* m, const void* E,
                    const uint32_t* beta, const uint32_t* v, size_t n_out, int phase2, void* stream);
/* one round of multi_hadamard_sumchecks (proof.cu:191-241) for K <= 4 tensors */
int zk_hadamard_round(uint32_t* coefs_host, void* const* new_Xs, const void* const* Xs, int K, const void* E, const uint32_t* v, size_t n_out, void* stream);
/* both sumchecks whole, queued without a host round trip (all rounds' sums come back in one copy): their challenges
 * are fixed before the first round (tLookup::prove tlookup.cu:150-176 and multi_hadamard_sumchecks proof.cu:191-241 take
 * u and v as arguments).  Rounds on short tensors (<= 512 pairs) run inside one launch.  Lookup: A, S of
 * D elements, B, T, m of N (D/N a power of two), E of D/2; v: rounds x 8 limbs in round order; sums_host: rounds x 11.
 * Hadamard: K tensors of N elements (a power of two), E of N/2; coefs_host: log2(N) x (K+1).  Inputs are not modified. */
int zk_lookup_sumcheck(uint32_t* sums_host, const void* A, const void* S, const void* B, const void* T, const void* m, const void* E, const uint32_t* beta,
                       const uint32_t* v, size_t D, size_t N, int rounds, void* stream);
int zk_hadamard_sumcheck(uint32_t* coefs_host, const void* const* Xs, int K, const void* E, const uint32_t* v, size_t N, void* stream);
/* the device side of a lookup proof / a multi-Hadamard proof as a job on a stream of the library's own, beside the
 * caller's stream (ordered after what `stream` holds at begin).  The lookup job also computes A = 1/(S+beta),
 * B = 1/(T+beta) (tlookup_inv_kernel tlookup.cu:337-352), <B, m> and the eq table of u_eq (rounds-1 challenges).
 * Inputs must stay alive and unmodified until end; every handle must be ended exactly once.  bm_host: <B, m>, 8 limbs. */
int zk_lookup_prove_begin(void** handle, const void* S, const void* T, const void* m, const uint32_t* beta, const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N,
                          int rounds, void* stream);
/* the same job when the queries are expected to be table entries (tLookupRange::prep / tLookupRangeMapping, tlookup.cu:393-421,
 * build S from the table): query i should equal T[hint[i] - low], hint being D field elements (for a range table the
 * looked-up values themselves).  Results are identical to zk_lookup_prove_begin's for every input; where the hint
 * holds, 1/(S[i]+beta) is read from B instead of being computed, and a query that does not match is inverted on its own. */
int zk_lookup_prove_begin_hinted(void** handle, const void* S, const void* T, const void* m, const void* hint_fr, int32_t low, const uint32_t* beta, const uint32_t* u_eq,
                                 const uint32_t* v, size_t D, size_t N, int rounds, void* stream);
/* the combined lookup of a mapping table (tLookupRangeMapping::prove, tlookup.cu:517-551): query i = S_in[i] + r * S_out[i], expected at
 * T[S_in[i] - low], T = table + r * mapped values; the combined queries are formed inside the first round instead of being written out */
int zk_lookup_prove_begin_mapped(void** handle, const void* S_in, const void* S_out, const uint32_t* r, const void* T, const void* m, int32_t low, const uint32_t* beta,
                                 const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N, int rounds, void* stream);
/* The two jobs above for queries that keep an int32 form (handles of zk_fr_fold_prepare / zk_fr_fold_prepared_new; the
 * tensors of field elements are given as well and serve the jobs too small for a fused first round).  _hinted_ints: the
 * queries S are their own hints (a range table's case, tLookupRange::prove, tlookup.cu:404-412).  _mapped_ints: S_in, S_out
 * and the table's mapped values (mapped_prepared: N integers, the padded mapped_vals of tLookupRangeMapping).  The first
 * round reads 4 bytes per query and tensor instead of 32 and takes query and inverse from the table wherever the table entry
 * at S_in[i] - low is what the integers say (checked per table entry on the device, so any T is safe); same results. */
/* 1 when a job of D queries into N entries reads its queries from their int32 forms alone: the tensors of field elements
 * passed beside them (S, S_in, S_out) are then never read and may be left unfilled (a padded copy need not be made) */
int zk_lookup_ints_suffice(size_t D, size_t N);
int zk_lookup_prove_begin_hinted_ints(void** handle, const void* S, const void* S_prepared, const void* T, const void* m, int32_t low, const uint32_t* beta,
                                      const uint32_t* u_eq, const uint32_t* v, size_t D, size_t N, int rounds, void* stream);
int zk_lookup_prove_begin_mapped_ints(void** handle, const void* S_in, const void* S_in_prepared, const void* S_out, const void* S_out_prepared, const void* mapped_prepared,
                                      const uint32_t* r, const void* T, const void* m, int32_t low, const uint32_t* beta, const uint32_t* u_eq, const uint32_t* v, size_t D,
                                      size_t N, int rounds, void* stream);
int zk_lookup_prove_end(void* handle, uint32_t* bm_host, uint32_t* sums_host);
/* Diagnostics of the job zk_lookup_prove_end collected last (no counterpart in the reference): *n_ok = how many leading table
 * entries were what the integers say -- the queries naming one of them took the first round's short path, the others their own
 * comparison -- and *n_table = the table's size; both 0 when the job had no int32 forms.  A range table of len entries padded to
 * a power of two by repeating its last value reports len.  ZKLLM_LOOKUP_TRUSTED=0 in the environment makes every job report 0:
 * each query is then compared on its own (same results; for comparing the two paths). */
int zk_lookup_last_job_consistent_entries(uint32_t* n_ok, uint32_t* n_table);
/* hadamard_product_sumcheck (Fr_hp_sc, proof.cu:66-109): adjacent-pair folding, first challenge first.  a, b: n elements,
 * 2^(k-1) < n <= 2^k; u, v: k challenges each.  proof_host: 3k + 2 values (per round the three terms evaluated at the
 * remaining u, then the folded a and b).  The three term tensors of the reference's step kernel are never materialised. */
int zk_hadamard_product_sumcheck(uint32_t* proof_host, const void* a, const void* b, const uint32_t* u, const uint32_t* v, size_t n, int k, void* stream);
/* the same in two halves: begin queues the rounds on a stream of the library's own, ordered behind what `stream` holds so far,
 * and returns at once (u and v are copied; a and b stay alive and unmodified until end); end waits and delivers the values */
int zk_hadamard_product_sumcheck_begin(void** handle, const void* a, const void* b, const uint32_t* u, const uint32_t* v, size_t n, int k, void* stream);
int zk_hadamard_product_sumcheck_end(void* handle, uint32_t* proof_host);
int zk_hadamard_prove_begin(void** handle, const void* const* Xs, int K, const uint32_t* u_eq, const uint32_t* v, size_t N, void* stream);
/* the same where prepareds[i], when non-null, is the int32 form of Xs[i] (N elements): two tensors that both have one (the
 * mapped outputs of a softmax's segments, zksoftmax.cu:177-180) are read from it in the first round; same sums */
int zk_hadamard_prove_begin_ints(void** handle, const void* const* Xs, const void* const* prepareds, int K, const uint32_t* u_eq, const uint32_t* v, size_t N, void* stream);
/* 1 when a job of zk_hadamard_prove_begin_ints over K tensors of N elements that all carry int32 forms reads nothing but those
 * forms (K == 2 and a job long enough to have a first round of its own): the field elements passed beside them need not hold
 * anything then.  No counterpart in the reference. */
int zk_hadamard_ints_suffice(int K, size_t N);
int zk_hadamard_prove_end(void* handle, uint32_t* coefs_host);

/* ---- rescaling / softmax ------------------------------------------------------------------------------------------ */
int zk_rescale(void* out, void* rem, const void* in, uint32_t scaling_factor, size_t n, void* stream);       /* rescaling_kernel rescaling.cu:8-21 */
/* the same, and rem_ints (int32, n) receives the remainders once more: they lie in [-sf/2, sf/2).  rem may be null where
 * rem_ints is given (here and in zk_rescale_ints_both): the remainders are written as int32 only */
int zk_rescale_ints(void* out, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* stream);
/* the same, and out_ints receives the rescaled values as int32; synchronises and reports in *out_fits_host whether every one
 * of them fits (0: out_ints must not be used) */
int zk_rescale_ints_both(void* out, void* out_ints, int* out_fits_host, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* stream);
/* the same with the answer left on the device: *bad_flag_dev (4 bytes of device memory) is cleared, then set by the kernel when a
 * rescaled value does not fit int32; the caller reads it (zk_memcpy_d2h) whenever the kernel is through and a wait costs nothing */
int zk_rescale_ints_both_flag(void* out, void* out_ints, void* bad_flag_dev, void* rem, void* rem_ints, const void* in, uint32_t scaling_factor, size_t n, void* stream);
int zk_i32_fill(void* dst_i32, int32_t value, size_t n, void* stream);       /* n int32 slots set to value (padding of an int32 form) */
/* zkrelu_decomp_kernel zkrelu.cu:8-29: the same rescaling, then sign (1 when the rescaled value is >= 0), magnitude and max(., 0) */
int zk_relu_decomp(void* res, void* sign, void* mag, void* rem, const void* in, uint32_t scaling_factor, size_t n, void* stream);
/* zksoftmax_shift zksoftmax.cu:20-32 (scale = sf_in*sqrt(d)), zksoftmax_calculate_table :4-14, zksoftmax_decompose_kernel :95-109 */
int zk_softmax_shift(void* shift, void* out_shifted, const void* X, uint32_t rows, uint32_t cols, double scale, void* stream);
int zk_softmax_table(void* table, double log_theta, double step, uint32_t len, void* stream);
/* planes: K device tensors of n elements each (host array of K pointers); plane k receives digit k */
int zk_softmax_decompose(void* const* planes, const void* X_shifted, const uint32_t* bs_host, int K, size_t n, void* stream);
/* the same, and int_planes[k] (int32, n each; null entries and a null array allowed) receive digit k once more as int32 */
int zk_softmax_decompose_ints(void* const* planes, void* const* int_planes, const void* X_shifted, const uint32_t* bs_host, int K, size_t n, void* stream);
/* zk_softmax_shift and zk_softmax_decompose_ints in one pass (zksoftmax.cu:124-140): the shifted scores are decomposed where
 * they are written, so they are not read again.  out_shifted may be null (the shifted scores are not written), and so may
 * planes[k] where int_planes[k] is given (digit k is written as int32 only). */
int zk_softmax_shift_decompose(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X, uint32_t rows, uint32_t cols, double scale,
                               const uint32_t* bs_host, int K, void* stream);
/* the same over scores given as 64-bit integers (rows * cols int64 on the device) */
int zk_softmax_shift_decompose_i64(void* shift, void* out_shifted, void* const* planes, void* const* int_planes, const void* X64, uint32_t rows, uint32_t cols, double scale,
                                   const uint32_t* bs_host, int K, void* stream);

/* ---- measurement helpers (no counterpart in the reference) ---------------------------------------- */
/* v_mad_u64_u32 issue peak of the device: 16 independent chains per lane, no memory traffic */
int zk_bench_mad_peak(uint32_t blocks, uint32_t iters, double* mad_per_s_host, void* stream);
/* plain 16-byte-per-lane copy of known size, to scale profiler byte counters */
int zk_bench_copy(void* dst, const void* src, size_t bytes, void* stream);
/* time the launches of the opening's fold kernel (the generator halving of me_open_step, commitment.cu:79-107) with
 * events on their stream: everything between begin and read.  fp_mults: base-field multiplications those launches
 * perform by the point formulas' count; pairs: generator pairs folded */
int zk_prof_fold_begin(void);
int zk_prof_fold_read(double* total_ms, unsigned long long* launches, double* fp_mults, unsigned long long* pairs);
/* what the last zk_prof_fold_read counted, split by fold method (three values each: the walk k_open_fold29, the combs
 * k_open_fold_comb<1> / <2>, the three-round fold k_open_fold_jump) */
int zk_prof_fold_methods(double* ms3, unsigned long long* launches3, unsigned long long* pairs3, double* fp_mults3);
/* the same for the int8-plane GEMM of the small-integer matrix products (k_gemm_i8_planes, behind zk_fr_matmul);
 * macs: int8 multiply-accumulates of those launches (rows x contraction x columns x plane pairs) */
int zk_prof_gemm_begin(void);
int zk_prof_gemm_read(double* total_ms, unsigned long long* launches, double* macs);
/* the same for the first round of the hinted lookup sumchecks (k_lookup_round<false, true>); bytes: their algorithmic traffic */
int zk_prof_lookup_begin(void);
int zk_prof_lookup_read(double* total_ms, unsigned long long* launches, unsigned long long* pairs, double* bytes);
/* and for the large rounds behind the first of every lookup sumcheck (phase 1, one lane per pair: k_lookup_round29), timed since
 * the same zk_prof_lookup_begin; bytes: 240 per pair (inverses and queries of both halves, eq weight, two folded values, next eq table) */
int zk_prof_lookup_later_read(double* total_ms, unsigned long long* launches, unsigned long long* pairs, double* bytes);

#ifdef __cplusplus
}
#endif
#endif

/*
 * tfo_oracle.h -- CPU restatement of tenferro's TensorPrims<Standard> operations and of the
 * pairwise einsum executor.  TEST INFRASTRUCTURE ONLY: it is the checker the HIP backend is
 * compared against and the timed CPU baseline; nothing in the shipped library links, loads or
 * calls it.
 *
 * The reference's own CPU backend is unimplemented (tenferro-prims/src/lib.rs:419-439 are
 * `todo!()`), so every function here follows the *documented formula* of the item it cites and
 * is pinned by the checks in tests/test_oracle.py and tests/test_golden.py (numpy cross-checks at
 * single-block and multi-block sizes, closed forms, brute force, the reference's doc examples,
 * exactly representable operands for the alpha/beta epilogue).  f32 products are accumulated in
 * f32 inside a cache block and in f64 across blocks: on outputs whose terms cancel the result
 * carries the rounding error of an f32 inner product (tests/golden/cancelling_f32.npz).  Numerical parity with a reference implementation is
 * therefore "parity unpinned": there is no reference implementation to compare with.
 */
#ifndef TFO_ORACLE_H
#define TFO_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define TFO_MAX_RANK 16
enum { TFO_F32 = 0, TFO_F64 = 1, TFO_C64 = 2, TFO_C128 = 3 };
enum { TFO_SUM = 0, TFO_MAX = 1, TFO_MIN = 2 };

/* Host strided view; same field order as the device view of the C ABI.
 * Element (i0,i1,..) lives at base + (offset + sum_d i_d*strides[d]) * sizeof(T)
 * (tenferro-tensor/src/lib.rs:169-171, 219-221). */
typedef struct tfo_view {
    void* base;
    int32_t rank;
    int32_t reserved;
    int64_t offset;
    int64_t dims[TFO_MAX_RANK];
    int64_t strides[TFO_MAX_RANK];
} tfo_view;

/* All functions return 0 on success, a negative number on invalid arguments
 * (-1 shape mismatch, -2 rank mismatch, -6 invalid argument), message in tfo_last_message(). */
const char* tfo_last_message(void);
int tfo_num_threads(void);
void tfo_set_num_threads(int n);

/* PrimDescriptor::Permute: B[modes_b] = alpha*A[modes_a] + beta*B  (tenferro-prims/src/lib.rs:194-202, 300-304) */
int tfo_permute(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
                const void* beta, tfo_view* b, const uint32_t* modes_b);
/* PrimDescriptor::Reduce: C[modes_c] = alpha*reduce_op(A[modes_a]) + beta*C  (:170-180, :100-107) */
int tfo_reduce(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
               const void* beta, tfo_view* c, const uint32_t* modes_c, int reduce_op);
/* PrimDescriptor::Contract: C[modes_c] = alpha*contract(A[modes_a],B[modes_b]) + beta*C
 * (:227-239; mode rule :136-138).  Cache-blocked, packed, multithreaded. */
int tfo_contract(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
                 const tfo_view* b, const uint32_t* modes_b,
                 const void* beta, tfo_view* c, const uint32_t* modes_c);
/* Same formula by brute force: one loop nest over every label, long-double accumulation.
 * Independent of tfo_contract; used to pin it.  Tiny shapes only. */
int tfo_contract_naive(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
                       const tfo_view* b, const uint32_t* modes_b,
                       const void* beta, tfo_view* c, const uint32_t* modes_c);
/* PrimDescriptor::BatchedGemm: C[batch,m,n] = alpha*A[batch,m,k]*B[batch,k,n] + beta*C  (:156-168).
 * Views have rank n_batch+2, batch axes first. */
int tfo_batched_gemm(int dtype, int n_batch, const void* alpha, const tfo_view* a, const tfo_view* b,
                     const void* beta, tfo_view* c);
/* PrimDescriptor::ElementwiseMul: C = alpha*A.*B + beta*C on same-shape views (:241-244). */
int tfo_elementwise_mul(int dtype, const void* alpha, const tfo_view* a, const tfo_view* b,
                        const void* beta, tfo_view* c);
/* PrimDescriptor::Trace: C[modes_c] = alpha*sum over the diagonal of every paired mode + beta*C (:182-192).
 * pairs = (i0,j0,i1,j1,..) mode labels; paired modes do not appear in modes_c. */
int tfo_trace(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
              const void* beta, tfo_view* c, const uint32_t* modes_c,
              const uint32_t* pairs, int n_pairs);
/* PrimDescriptor::AntiTrace (:204-212): C[modes_c] = alpha*A[modes_a] placed on the diagonal
 * i==j of every pair (zero elsewhere) + beta*C; the adjoint of Trace.  modes_c holds both i and j. */
int tfo_anti_trace(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
                   const void* beta, tfo_view* c, const uint32_t* modes_c,
                   const uint32_t* pairs, int n_pairs);
/* PrimDescriptor::AntiDiag (:214-222): like AntiTrace but A still carries mode i of each pair
 * (the adjoint of diagonal extraction "ii->i"). */
int tfo_anti_diag(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a,
                  const void* beta, tfo_view* c, const uint32_t* modes_c,
                  const uint32_t* pairs, int n_pairs);
/* Tensor::conj (tenferro-tensor/src/lib.rs:622-647): negate the imaginary part; copy for reals. */
int tfo_conj(int dtype, const tfo_view* in, tfo_view* out);

/* einsum by brute force over every label (tenferro-einsum/src/lib.rs:37-93 pattern catalogue:
 * repeated labels in an operand take its diagonal, labels repeated in the output write a
 * diagonal, labels absent from the output are summed).  out = alpha*einsum + beta*out.
 * labels: concatenated operand labels; ranks[i] = rank of operand i. */
int tfo_einsum_naive(int dtype, int n_inputs, const tfo_view* inputs, const uint32_t* labels,
                     const int32_t* ranks, const uint32_t* out_labels, int n_out,
                     const void* alpha, const void* beta, tfo_view* out);
/* einsum along a given pairwise order (ContractionTree::from_pairs numbering,
 * tenferro-einsum/src/lib.rs:320-355), each step through tfo_contract, intermediates row-major.
 * Operands must not repeat a label internally.  pairs holds 2*n_pairs indices. */
int tfo_einsum_pairs(int dtype, int n_inputs, const tfo_view* inputs, const uint32_t* labels,
                     const int32_t* ranks, const uint32_t* out_labels, int n_out,
                     const int32_t* pairs, int n_pairs,
                     const void* alpha, const void* beta, tfo_view* out);

#ifdef __cplusplus
}
#endif
#endif

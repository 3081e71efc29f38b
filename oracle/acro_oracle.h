/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * CPU restatement, in plain C, of the reference's host execution path: the "CPUInterpreted" policy and the
 * NativeCPUOps non-contraction operations.  It is the checker that tests, the smoke test and the benchmark's
 * cpu_baseline leg compare the HIP backend against; nothing in the product library links or calls it.
 *
 * Every function names the reference code it follows.  What pins each function:
 *  - all of them: bit-exact agreement with the compiled reference (oracle/_ref, built from /root/reference by
 *    oracle/Makefile) on seeded random inputs (tests/test_oracle_vs_reference.py) and against the golden
 *    fixtures that the compiled reference wrote (tests/golden);
 *  - contraction: brute-force numpy einsum on integer-valued data (exact), textbook special cases (matvec,
 *    transpose, trace, diagonal) and the known-answer cases of the reference's unittest/kernel/test_TensorEngine.cpp;
 *  - inverse / determinant: A * inv(A)^T = I (3x3), A * inv(A) = I (2x2), det(A) det(inv A) = 1;
 *  - scatter / gather: the 8 -> 6 example of unittest/kernel/test_TensorEngine.cpp:708-745.
 * No function is "parity unpinned".
 */
#ifndef ACRO_ORACLE_H
#define ACRO_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ACRO_ORACLE_MAX_VARS 16
#define ACRO_ORACLE_MAX_RANK 16
#define ACRO_ORACLE_MAX_IDX 32
#define ACRO_ORACLE_NAME_LEN 32

typedef struct
{
    char name[ACRO_ORACLE_NAME_LEN];
    int rank;
    char index[ACRO_ORACLE_MAX_RANK][ACRO_ORACLE_NAME_LEN];
} acro_oracle_var;

typedef struct
{
    acro_oracle_var out;
    char op[3]; /* "=", "+=" or "-=" */
    int num_in;
    acro_oracle_var in[ACRO_ORACLE_MAX_VARS];
    int num_idx;       /* all indices: output indices first, then contraction indices by first appearance */
    int num_outer;     /* how many of them belong to the output */
    char idx[ACRO_ORACLE_MAX_IDX][ACRO_ORACLE_NAME_LEN];
} acro_oracle_kernel;

/* Grammar of kernel/TensorKernel.cpp:26-139.  Returns 0 on success, non-zero where the reference asserts. */
int acro_oracle_parse(const char *kernel_str, acro_oracle_kernel *k);

/* "Out_i_j" + eq|pe|me + "In_..."  (kernel/TensorKernel.cpp:327-357); returns 0 on success. */
int acro_oracle_name_string(const char *kernel_str, char *buf, size_t buflen);

/*
 * One contraction exactly as CPUInterpretedExecutor::ExecuteSingle runs it
 * (exec/CPUInterpretedExecutor.cpp:59-91,99-444 with the inner statement of .hpp:58-77):
 * "=" zero-fills the output first; then for every index combination, outer indices outermost and contraction
 * indices innermost in first-appearance order, out[..] += in0[..] * in1[..] * ... (product left to right).
 * "-=" ADDS, like the reference's interpreter (its loop bodies only ever use +=).
 * dims[v] holds the extents of variable v (v = 0 is the output, then the inputs in order).
 * Returns 0, or non-zero with a message in err for a parse error, a rank mismatch or incompatible extents.
 */
int acro_oracle_contract(const char *kernel_str, double *out, const double *const *ins, int num_in,
                         const int *const *dims, const int *ranks, char *err, size_t errlen);

/* ops/NativeCPUOps.hpp:38-86 and ops/NativeCPUOps.cpp:11-123; mdim in {1,2,3}; returns non-zero otherwise. */
int acro_oracle_batch_matrix_inverse(double *Ainv, const double *A, int mdim, long num_batch);
int acro_oracle_batch_matrix_det(double *Adet, const double *A, int mdim, long num_batch);
int acro_oracle_batch_matrix_inv_det(double *Ainv, double *Adet, const double *A, int mdim, long num_batch);

/* ops/NativeCPUOps.cpp:126-144 */
void acro_oracle_flat_indexed_scatter(double *Aout, const double *Ain, const int *M, int range_size);
void acro_oracle_flat_indexed_sum_gather(double *Aout, int domain_size, const double *Ain, const int *M,
                                         int range_size);

/* tensor/IndexMapping.cpp:27-51: inverse map (range entries stably ordered by image) and row offsets, computed
 * with the reference's own offset walk. */
void acro_oracle_index_mapping_inverse(const int *M, int domain_size, int range_size, int *InvM, int *InvMOff);

#ifdef __cplusplus
}
#endif

#endif

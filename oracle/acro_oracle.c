/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.  See acro_oracle.h.
 * Plain-C restatement of the reference's CPU path; compiled with -ffp-contract=off so that every multiply and add
 * rounds separately, as the reference built with g++ for x86-64 does.
 */
#include "acro_oracle.h"

#include <ctype.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ parsing */

static int is_idx_char(char c)
{
    return islower((unsigned char)c) || isdigit((unsigned char)c);
}

/* var := NAME ('_' IDX)+ ; NAME := [A-Z][A-Za-z0-9]* ; IDX := [a-z0-9]+   (kernel/TensorKernel.cpp:70-117) */
static int parse_var(const char **pp, acro_oracle_var *v)
{
    const char *p = *pp;
    int n = 0;
    memset(v, 0, sizeof(*v));
    if (!isupper((unsigned char)*p)) return 1;
    while (isalnum((unsigned char)*p))
    {
        if (n + 1 >= ACRO_ORACLE_NAME_LEN) return 1;
        v->name[n++] = *p++;
    }
    if (*p != '_') return 1;
    while (*p == '_')
    {
        int m = 0;
        ++p;
        if (!is_idx_char(*p)) return 1;
        if (v->rank >= ACRO_ORACLE_MAX_RANK) return 1;
        while (is_idx_char(*p))
        {
            if (m + 1 >= ACRO_ORACLE_NAME_LEN) return 1;
            v->index[v->rank][m++] = *p++;
        }
        v->rank++;
    }
    *pp = p;
    return 0;
}

static int find_idx(const acro_oracle_kernel *k, const char *name)
{
    int i;
    for (i = 0; i < k->num_idx; ++i)
        if (strcmp(k->idx[i], name) == 0) return i;
    return -1;
}

int acro_oracle_parse(const char *kernel_str, acro_oracle_kernel *k)
{
    char *text = (char *)malloc(strlen(kernel_str) + 1);
    const char *p;
    int n = 0, v, d, rc = 1;
    if (text == NULL) return 1;
    /* all white space is removed first (kernel/TensorKernel.cpp:31) */
    for (p = kernel_str; *p; ++p)
        if (!isspace((unsigned char)*p)) text[n++] = *p;
    text[n] = '\0';
    memset(k, 0, sizeof(*k));

    p = text;
    if (parse_var(&p, &k->out)) goto done;
    if (*p == '=')
    {
        strcpy(k->op, "=");
        p += 1;
    }
    else if ((*p == '+' || *p == '-') && p[1] == '=')
    {
        k->op[0] = *p;
        k->op[1] = '=';
        p += 2;
    }
    else
        goto done;
    do
    {
        if (k->num_in >= ACRO_ORACLE_MAX_VARS) goto done;
        if (parse_var(&p, &k->in[k->num_in])) goto done;
        k->num_in++;
    } while (*p);

    /* output indices first, then unseen input indices in order of appearance (kernel/TensorKernel.cpp:46-63) */
    for (d = 0; d < k->out.rank; ++d)
    {
        if (find_idx(k, k->out.index[d]) < 0)
        {
            if (k->num_idx >= ACRO_ORACLE_MAX_IDX) goto done;
            strcpy(k->idx[k->num_idx++], k->out.index[d]);
        }
    }
    k->num_outer = k->num_idx;
    for (v = 0; v < k->num_in; ++v)
    {
        for (d = 0; d < k->in[v].rank; ++d)
        {
            if (find_idx(k, k->in[v].index[d]) < 0)
            {
                if (k->num_idx >= ACRO_ORACLE_MAX_IDX) goto done;
                strcpy(k->idx[k->num_idx++], k->in[v].index[d]);
            }
        }
    }
    rc = 0;
done:
    free(text);
    return rc;
}

int acro_oracle_name_string(const char *kernel_str, char *buf, size_t buflen)
{
    acro_oracle_kernel k;
    int v, d;
    size_t used = 0;
    if (acro_oracle_parse(kernel_str, &k)) return 1;
#define APPEND(s)                                          \
    do                                                     \
    {                                                      \
        size_t l_ = strlen(s);                             \
        if (used + l_ + 1 > buflen) return 2;              \
        memcpy(buf + used, s, l_);                         \
        used += l_;                                        \
        buf[used] = '\0';                                  \
    } while (0)
    APPEND(k.out.name);
    for (d = 0; d < k.out.rank; ++d)
    {
        APPEND("_");
        APPEND(k.out.index[d]);
    }
    APPEND(k.op[0] == '=' ? "eq" : (k.op[0] == '+' ? "pe" : "me"));
    for (v = 0; v < k.num_in; ++v)
    {
        APPEND(k.in[v].name);
        for (d = 0; d < k.in[v].rank; ++d)
        {
            APPEND("_");
            APPEND(k.in[v].index[d]);
        }
    }
#undef APPEND
    return 0;
}

/* -------------------------------------------------------------------------------------- contraction */

int acro_oracle_contract(const char *kernel_str, double *out, const double *const *ins, int num_in,
                         const int *const *dims, const int *ranks, char *err, size_t errlen)
{
    acro_oracle_kernel k;
    int extent[ACRO_ORACLE_MAX_IDX];
    /* element stride of every variable (0 = output) with respect to every loop index */
    long stride[ACRO_ORACLE_MAX_VARS + 1][ACRO_ORACLE_MAX_IDX];
    int I[ACRO_ORACLE_MAX_IDX];
    int v, d, i, nloops;
    long out_size = 1;

#define FAIL(msg)                                           \
    do                                                      \
    {                                                       \
        if (err && errlen) snprintf(err, errlen, "%s", msg); \
        return 1;                                           \
    } while (0)

    if (acro_oracle_parse(kernel_str, &k)) FAIL("kernel string does not parse");
    if (num_in != k.num_in) FAIL("number of input tensors does not match the kernel");
    nloops = k.num_idx;
    for (i = 0; i < nloops; ++i) extent[i] = 0;
    memset(stride, 0, sizeof(stride));

    /* extents from the tensors; every use of an index must agree (kernel/TensorKernel.cpp:375-403) */
    for (v = 0; v <= k.num_in; ++v)
    {
        const acro_oracle_var *var = (v == 0) ? &k.out : &k.in[v - 1];
        long st = 1;
        if (ranks[v] != var->rank) FAIL("tensor rank does not match the kernel variable");
        for (d = var->rank - 1; d >= 0; --d)
        {
            int li = find_idx(&k, var->index[d]);
            if (dims[v][d] <= 0) FAIL("non-positive tensor extent");
            if (extent[li] != 0 && extent[li] != dims[v][d]) FAIL("Incompatible tensor dimensions for kernel");
            extent[li] = dims[v][d];
            /* row-major strides from the extents (kernel/DimensionedKernel.cpp:133-145); an index used twice in
             * one variable ("B_i_i") accumulates both strides, as ComputeRawIdx does (exec/..Executor.hpp:69-77) */
            stride[v][li] += st;
            st *= dims[v][d];
        }
        if (v == 0) out_size = st;
    }

    /* "=" is zero-fill followed by accumulation (exec/CPUInterpretedExecutor.cpp:63-67) */
    if (k.op[0] == '=')
    {
        long n;
        for (n = 0; n < out_size; ++n) out[n] = 0.0;
    }

    /* odometer over all loops: outer indices first, contraction indices innermost, last index fastest
     * (exec/CPUInterpretedExecutor.cpp:99-444).  The reference orders the outer loops by extent
     * (kernel/DimensionedMultiKernel.cpp:91-134); that order does not change any sum because every output entry
     * receives its terms in contraction order either way. */
    for (i = 0; i < nloops; ++i) I[i] = 0;
    {
        /* running element offsets of every variable, updated as the odometer turns */
        long off[ACRO_ORACLE_MAX_VARS + 1];
        for (v = 0; v <= k.num_in; ++v) off[v] = 0;
        for (;;)
        {
            double rhs = ins[0][off[1]];
            for (v = 2; v <= k.num_in; ++v) rhs *= ins[v - 1][off[v]];
            out[off[0]] += rhs; /* also for "-=": the reference interpreter never subtracts */

            for (i = nloops - 1; i >= 0; --i)
            {
                if (++I[i] < extent[i])
                {
                    for (v = 0; v <= k.num_in; ++v) off[v] += stride[v][i];
                    break;
                }
                I[i] = 0;
                for (v = 0; v <= k.num_in; ++v) off[v] -= (long)(extent[i] - 1) * stride[v][i];
            }
            if (i < 0) break;
        }
    }
#undef FAIL
    return 0;
}

/* ---------------------------------------------------------------------------- small matrix operations */

/* ops/NativeCPUOps.hpp:72-86 */
static double det1(const double *A) { return A[0]; }
static double det2(const double *A) { return (A[0] * A[3] - A[1] * A[2]); }
static double det3(const double *A)
{
    return (A[0] * A[4] * A[8] + A[1] * A[5] * A[6] + A[2] * A[3] * A[7] - A[6] * A[4] * A[2] - A[7] * A[5] * A[0] -
            A[8] * A[3] * A[1]);
}

/* ops/NativeCPUOps.hpp:38-67.  The 3x3 result is the cofactor matrix over the determinant WITHOUT the final
 * transposition, i.e. the transpose of the inverse for a non-symmetric matrix - the reference does exactly this. */
static void inv1(double *R, const double *A, double det)
{
    (void)A;
    R[0] = 1.0 / det;
}
static void inv2(double *R, const double *A, double det)
{
    double invdet = 1.0 / det;
    R[0] = invdet * A[3];
    R[1] = -invdet * A[1];
    R[2] = -invdet * A[2];
    R[3] = invdet * A[0];
}
static void inv3(double *R, const double *A, double det)
{
    double invdet = 1.0 / det;
    R[0] = invdet * (A[4] * A[8] - A[5] * A[7]);
    R[1] = invdet * (A[5] * A[6] - A[3] * A[8]);
    R[2] = invdet * (A[3] * A[7] - A[4] * A[6]);
    R[3] = invdet * (A[2] * A[7] - A[1] * A[8]);
    R[4] = invdet * (A[0] * A[8] - A[2] * A[6]);
    R[5] = invdet * (A[1] * A[6] - A[0] * A[7]);
    R[6] = invdet * (A[1] * A[5] - A[2] * A[4]);
    R[7] = invdet * (A[2] * A[3] - A[0] * A[5]);
    R[8] = invdet * (A[0] * A[4] - A[1] * A[3]);
}

static double det_of(const double *A, int mdim)
{
    return mdim == 1 ? det1(A) : (mdim == 2 ? det2(A) : det3(A));
}

static void inv_of(double *R, const double *A, double det, int mdim)
{
    if (mdim == 1)
        inv1(R, A, det);
    else if (mdim == 2)
        inv2(R, A, det);
    else
        inv3(R, A, det);
}

int acro_oracle_batch_matrix_inverse(double *Ainv, const double *A, int mdim, long num_batch)
{
    long i;
    int mm = mdim * mdim;
    if (mdim < 1 || mdim > 3) return 1;
    for (i = 0; i < num_batch; ++i) inv_of(Ainv + i * mm, A + i * mm, det_of(A + i * mm, mdim), mdim);
    return 0;
}

int acro_oracle_batch_matrix_det(double *Adet, const double *A, int mdim, long num_batch)
{
    long i;
    int mm = mdim * mdim;
    if (mdim < 1 || mdim > 3) return 1;
    for (i = 0; i < num_batch; ++i) Adet[i] = det_of(A + i * mm, mdim);
    return 0;
}

int acro_oracle_batch_matrix_inv_det(double *Ainv, double *Adet, const double *A, int mdim, long num_batch)
{
    long i;
    int mm = mdim * mdim;
    if (mdim < 1 || mdim > 3) return 1;
    for (i = 0; i < num_batch; ++i)
    {
        Adet[i] = det_of(A + i * mm, mdim);
        inv_of(Ainv + i * mm, A + i * mm, Adet[i], mdim);
    }
    return 0;
}

/* ------------------------------------------------------------------------------ indexed copy and sum */

void acro_oracle_flat_indexed_scatter(double *Aout, const double *Ain, const int *M, int range_size)
{
    int i;
    for (i = 0; i < range_size; ++i) Aout[i] = Ain[M[i]];
}

void acro_oracle_flat_indexed_sum_gather(double *Aout, int domain_size, const double *Ain, const int *M,
                                         int range_size)
{
    int i;
    for (i = 0; i < domain_size; ++i) Aout[i] = 0.0;
    for (i = 0; i < range_size; ++i) Aout[M[i]] += Ain[i];
}

void acro_oracle_index_mapping_inverse(const int *M, int domain_size, int range_size, int *InvM, int *InvMOff)
{
    /* stable ordering of the range entries by their image: insertion into counting buckets keeps range order */
    int i, off;
    int *count = (int *)calloc((size_t)domain_size + 1, sizeof(int));
    for (i = 0; i < range_size; ++i) count[M[i] + 1]++;
    for (i = 0; i < domain_size; ++i) count[i + 1] += count[i];
    for (i = 0; i < range_size; ++i) InvM[count[M[i]]++] = i;
    free(count);

    /* the reference's offset walk (tensor/IndexMapping.cpp:35-51): each row takes the next run of equal images,
     * so rows stay aligned with domain entries only when every domain entry has a preimage */
    off = 0;
    for (i = 0; i < domain_size + 1; ++i)
    {
        InvMOff[i] = off;
        if (off < range_size)
        {
            int m = M[InvM[off]];
            while (off < range_size && M[InvM[off]] == m) off++;
        }
        else
        {
            off = range_size;
        }
    }
}

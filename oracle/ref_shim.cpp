// TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
// C shim over the reference library itself (compiled from the sources under /root/reference by the Makefile next
// to this file, CPU policy only).  It exposes the same C signatures as acro_oracle.h with the prefix acro_ref_,
// so that tests can check the plain-C restatement against the real reference bit for bit, and so that the
// benchmark can time the reference's own CPUInterpreted executor as the CPU baseline.
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "AcroTensor.hpp"

using namespace acro;

namespace
{
std::vector<int> toVec(const int *d, int n)
{
    return std::vector<int>(d, d + n);
}

int fail(char *err, size_t errlen, const char *msg)
{
    if (err && errlen) snprintf(err, errlen, "%s", msg);
    return 1;
}
}  // namespace

extern "C" {

// TensorEngine("CPUInterpreted")(kernel, out, inputs) on caller-owned buffers
int acro_ref_contract(const char *kernel_str, double *out, const double *const *ins, int num_in,
                      const int *const *dims, const int *ranks, char *err, size_t errlen)
{
    try
    {
        TensorEngine TE("CPUInterpreted");
        std::vector<int> od = toVec(dims[0], ranks[0]);
        Tensor O(od, out);
        std::vector<Tensor *> in;
        std::vector<Tensor *> owned;
        for (int v = 0; v < num_in; ++v)
        {
            std::vector<int> d = toVec(dims[v + 1], ranks[v + 1]);
            owned.push_back(new Tensor(d, const_cast<double *>(ins[v])));
            in.push_back(owned.back());
        }
        std::string ks(kernel_str);
        int rc = 0;
        try
        {
            TE(ks, &O, in);
        }
        catch (const std::exception &ex)
        {
            rc = fail(err, errlen, ex.what());
        }
        for (Tensor *t : owned) delete t;
        return rc;
    }
    catch (const std::exception &ex)
    {
        return fail(err, errlen, ex.what());
    }
}

// A whole multi-kernel launch (Begin/EndMultiKernelLaunch) on the CPU policy.  tensors are listed per kernel,
// output first; tensor_ids name them so that one buffer can appear in several kernels.
int acro_ref_multi_contract(int num_kernels, const char *const *kernels, const int *num_in, double *const *buffers,
                            const int *const *dims, const int *ranks, char *err, size_t errlen)
{
    try
    {
        TensorEngine TE("CPUInterpreted");
        std::vector<Tensor *> owned;
        TE.BeginMultiKernelLaunch();
        int t = 0;
        for (int k = 0; k < num_kernels; ++k)
        {
            std::vector<Tensor *> list;
            for (int v = 0; v <= num_in[k]; ++v, ++t)
            {
                std::vector<int> d = toVec(dims[t], ranks[t]);
                owned.push_back(new Tensor(d, buffers[t]));
                list.push_back(owned.back());
            }
            Tensor *O = list[0];
            std::vector<Tensor *> in(list.begin() + 1, list.end());
            std::string ks(kernels[k]);
            TE(ks, O, in);
        }
        TE.EndMultiKernelLaunch();
        for (Tensor *p : owned) delete p;
        return 0;
    }
    catch (const std::exception &ex)
    {
        return fail(err, errlen, ex.what());
    }
}

int acro_ref_name_string(const char *kernel_str, char *buf, size_t buflen)
{
    try
    {
        TensorKernel k(kernel_str);
        std::string s = k.GetNameString();
        if (s.size() + 1 > buflen) return 2;
        std::memcpy(buf, s.c_str(), s.size() + 1);
        return 0;
    }
    catch (const std::exception &)
    {
        return 1;
    }
}

// Text description of the parse and of the single-kernel loop order after binding to shapes:
// "all:i,j,k;contr:k;loops:i,j,k;dims:3,4,5;dname:<dimensioned name>"
int acro_ref_describe(const char *kernel_str, const int *const *dims, const int *ranks, int num_in, char *buf,
                      size_t buflen)
{
    try
    {
        TensorKernel k(kernel_str);
        std::vector<double> dummy(1);
        std::vector<int> od = toVec(dims[0], ranks[0]);
        Tensor O(od, dummy.data());
        std::vector<Tensor *> in;
        for (int v = 0; v < num_in; ++v)
        {
            std::vector<int> d = toVec(dims[v + 1], ranks[v + 1]);
            in.push_back(new Tensor(d, dummy.data()));
        }
        DimensionedKernel dk(&k, &O, in);
        std::string dname1 = k.GetDimensionedNameString(&O, in);
        std::string dname2 = dk.GetDimensionedNameString();
        DimensionedMultiKernel mk(&dk);
        std::string s = "all:";
        for (size_t i = 0; i < k.AllIndexNames.size(); ++i) s += (i ? "," : "") + k.AllIndexNames[i];
        s += ";contr:";
        for (size_t i = 0; i < k.ContractionIndexNames.size(); ++i) s += (i ? "," : "") + k.ContractionIndexNames[i];
        s += ";loops:";
        for (size_t i = 0; i < mk.LoopIndices.size(); ++i) s += (i ? "," : "") + mk.LoopIndices[i];
        s += ";dims:";
        for (int i = 0; i < mk.GetNumIndices(); ++i) s += (i ? "," : "") + std::to_string(mk.GetLoopDim(i));
        s += ";dname:" + dname1 + ";dname2:" + dname2;
        s += ";flat:" + std::to_string(dk.GetFlatIdxSize()) + ";out:" + std::to_string(dk.GetOutIdxSize()) +
             ";cont:" + std::to_string(dk.GetContIdxSize());
        for (Tensor *t : in) delete t;
        if (s.size() + 1 > buflen) return 2;
        std::memcpy(buf, s.c_str(), s.size() + 1);
        return 0;
    }
    catch (const std::exception &)
    {
        return 1;
    }
}

static Tensor *wrapBatch(double *p, int mdim, long num_batch, bool matrix)
{
    std::vector<int> d;
    d.push_back(static_cast<int>(num_batch));
    if (matrix)
    {
        d.push_back(mdim);
        d.push_back(mdim);
    }
    return new Tensor(d, p);
}

int acro_ref_batch_matrix_inverse(double *Ainv, const double *A, int mdim, long num_batch)
{
    try
    {
        TensorEngine TE("CPUInterpreted");
        Tensor *a = wrapBatch(const_cast<double *>(A), mdim, num_batch, true);
        Tensor *r = wrapBatch(Ainv, mdim, num_batch, true);
        TE.BatchMatrixInverse(*r, *a);
        delete a;
        delete r;
        return 0;
    }
    catch (const std::exception &)
    {
        return 1;
    }
}

int acro_ref_batch_matrix_det(double *Adet, const double *A, int mdim, long num_batch)
{
    try
    {
        TensorEngine TE("CPUInterpreted");
        Tensor *a = wrapBatch(const_cast<double *>(A), mdim, num_batch, true);
        Tensor *r = wrapBatch(Adet, mdim, num_batch, false);
        TE.BatchMatrixDet(*r, *a);
        delete a;
        delete r;
        return 0;
    }
    catch (const std::exception &)
    {
        return 1;
    }
}

int acro_ref_batch_matrix_inv_det(double *Ainv, double *Adet, const double *A, int mdim, long num_batch)
{
    try
    {
        TensorEngine TE("CPUInterpreted");
        Tensor *a = wrapBatch(const_cast<double *>(A), mdim, num_batch, true);
        Tensor *r = wrapBatch(Ainv, mdim, num_batch, true);
        Tensor *dt = wrapBatch(Adet, mdim, num_batch, false);
        TE.BatchMatrixInvDet(*r, *dt, *a);
        delete a;
        delete r;
        delete dt;
        return 0;
    }
    catch (const std::exception &)
    {
        return 1;
    }
}

void acro_ref_flat_indexed_scatter(double *Aout, const double *Ain, int domain_size, const int *M, int range_size)
{
    TensorEngine TE("CPUInterpreted");
    IndexMapping map(domain_size, range_size);
    for (int i = 0; i < range_size; ++i) map[i] = M[i];
    Tensor out(range_size, Aout), in(domain_size, const_cast<double *>(Ain));
    TE.FlatIndexedScatter(out, in, map);
}

void acro_ref_flat_indexed_sum_gather(double *Aout, int domain_size, const double *Ain, const int *M, int range_size)
{
    TensorEngine TE("CPUInterpreted");
    IndexMapping map(domain_size, range_size);
    for (int i = 0; i < range_size; ++i) map[i] = M[i];
    Tensor out(domain_size, Aout), in(range_size, const_cast<double *>(Ain));
    TE.FlatIndexedSumGather(out, in, map);
}

void acro_ref_index_mapping_inverse(const int *M, int domain_size, int range_size, int *InvM, int *InvMOff)
{
    IndexMapping map(domain_size, range_size);
    for (int i = 0; i < range_size; ++i) map[i] = M[i];
    map.ComputeInverse();
    for (int i = 0; i < range_size; ++i) InvM[i] = map.GetInvMap()[i];
    for (int i = 0; i < domain_size + 1; ++i) InvMOff[i] = map.GetInvMapOffsets()[i];
}

}  // extern "C"

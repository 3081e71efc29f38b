// acro::NonContractionOps — batched small-matrix and indexed copy operations that are not tensor contractions
// (interface of the reference's ops/NonContractionOps.hpp:17-32).  Callers validate shapes and residency
// (TensorEngine); implementations trust their arguments.
#ifndef ACRO_HIP_NON_CONTRACTION_OPS_HPP
#define ACRO_HIP_NON_CONTRACTION_OPS_HPP

#include "IndexMapping.hpp"
#include "Tensor.hpp"

namespace acro
{

class NonContractionOps
{
  public:
    virtual ~NonContractionOps() {}
    // Batched 1x1, 2x2 and 3x3 matrices in the two trailing dimensions; all leading dimensions are batch.
    // For 3x3 the "inverse" is the cofactor matrix divided by the determinant laid out without the final
    // transposition, exactly as the reference computes it (ops/NativeCPUOps.hpp:55-67).
    virtual void BatchMatrixInverse(Tensor &Ainv, Tensor &A) = 0;
    virtual void BatchMatrixDet(Tensor &Adet, Tensor &A) = 0;
    virtual void BatchMatrixInvDet(Tensor &Ainv, Tensor &Adet, Tensor &A) = 0;
    // Aout[i] = Ain[M[i]] for i in the range of M
    virtual void FlatIndexedScatter(Tensor &Aout, Tensor &Ain, IndexMapping &M) = 0;
    // Aout[:] = 0; Aout[M[i]] += Ain[i] in increasing i
    virtual void FlatIndexedSumGather(Tensor &Aout, Tensor &Ain, IndexMapping &M) = 0;
};

// The "HIP" implementation (replaces the reference's ops/CudaGPUOps.{hpp,cpp}); operands are device resident.
class HipGPUOps : public NonContractionOps
{
  public:
    void BatchMatrixInverse(Tensor &Ainv, Tensor &A) override;
    void BatchMatrixDet(Tensor &Adet, Tensor &A) override;
    void BatchMatrixInvDet(Tensor &Ainv, Tensor &Adet, Tensor &A) override;
    void FlatIndexedScatter(Tensor &Aout, Tensor &Ain, IndexMapping &M) override;
    void FlatIndexedSumGather(Tensor &Aout, Tensor &Ain, IndexMapping &M) override;
};

}  // namespace acro

#endif

// acro::IndexMapping — a map M from a range of size RangeSize into a domain of size DomainSize, plus its
// inverse in compressed-row form (InvM sorted stably by M, InvMOff[d]..InvMOff[d+1] delimiting the range entries
// that map to domain entry d).  Reference: tensor/IndexMapping.hpp:13-45, tensor/IndexMapping.cpp:14-135.
#ifndef ACRO_HIP_INDEXMAPPING_HPP
#define ACRO_HIP_INDEXMAPPING_HPP

#include "IndexVector.hpp"

namespace acro
{

class IndexMapping
{
  public:
    IndexMapping(int domain_size, int range_size);

    int GetDomainSize() const { return DomainSize; }
    int GetRangeSize() const { return RangeSize; }
    bool IsInverseComputed() const { return InverseComputed; }

    int &operator[](int raw_index) { return M[raw_index]; }
    void ComputeInverse();

    IndexVector &GetMap() { return M; }
    IndexVector &GetInvMap();
    IndexVector &GetInvMapOffsets();

    void MapToGPU();
    void MoveToGPU();
    void SwitchToGPU();
    void UnmapFromGPU();
    void MoveFromGPU();
    void SwitchFromGPU();
    bool IsMappedToGPU() const { return MappedToGPU; }
    bool IsOnGPU() const { return OnGPU; }

  private:
    bool InverseComputed;
    bool MappedToGPU;
    bool OnGPU;
    int DomainSize;
    int RangeSize;
    IndexVector M;
    IndexVector InvM, InvMOff;
};

}  // namespace acro

#endif
